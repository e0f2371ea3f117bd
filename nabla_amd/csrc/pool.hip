// max_pool2d and avg_pool2d forward / backward over NHWC.  Lanes run along C (coalesced).
// max: windows are clipped at the padded border; the backward pass gives the full
// cotangent of a window to every element equal to that window's maximum.
// avg: the padding counts as zeros and every window is divided by kh * kw.
#include "nbk_common.h"

__global__ __launch_bounds__(256) void maxpool_fwd_kernel(const void* __restrict__ x,
                                                          void* __restrict__ y, nbk_pool_desc d) {
  const int64_t total = d.N * d.Ho * d.Wo * d.C;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int64_t c = i % d.C;
    int64_t t = i / d.C;
    const int64_t wo = t % d.Wo; t /= d.Wo;
    const int64_t ho = t % d.Ho;
    const int64_t n = t / d.Ho;
    const int64_t h0 = max((int64_t)0, ho * d.stride_h - d.pad_t);
    const int64_t h1 = min(d.H, ho * d.stride_h - d.pad_t + d.kh);
    const int64_t w0 = max((int64_t)0, wo * d.stride_w - d.pad_l);
    const int64_t w1 = min(d.W, wo * d.stride_w - d.pad_l + d.kw);
    float m = -INFINITY;
    for (int64_t h = h0; h < h1; ++h)
      for (int64_t w = w0; w < w1; ++w)
        m = fmaxf(m, nbk_load_as_f32(x, ((n * d.H + h) * d.W + w) * d.C + c, d.dtype));
    nbk_store_from_f32(y, i, d.dtype, m);
  }
}

__global__ __launch_bounds__(256) void maxpool_bwd_kernel(const void* __restrict__ x,
                                                          const void* __restrict__ y,
                                                          const void* __restrict__ dy,
                                                          void* __restrict__ dx, nbk_pool_desc d) {
  // gather form: each input element sums the cotangents of the windows that
  // contain it and whose maximum it equals -- no atomics, deterministic.
  const int64_t total = d.N * d.H * d.W * d.C;
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int64_t c = i % d.C;
    int64_t t = i / d.C;
    const int64_t w = t % d.W; t /= d.W;
    const int64_t h = t % d.H;
    const int64_t n = t / d.H;
    const float xv = nbk_load_as_f32(x, i, d.dtype);
    // windows ho with ho*sh - pt <= h < ho*sh - pt + kh
    const int64_t hp = h + d.pad_t, wp = w + d.pad_l;
    int64_t ho_lo = hp - d.kh + 1;
    ho_lo = ho_lo <= 0 ? 0 : (ho_lo + d.stride_h - 1) / d.stride_h;
    const int64_t ho_hi = min(d.Ho - 1, hp / d.stride_h);
    int64_t wo_lo = wp - d.kw + 1;
    wo_lo = wo_lo <= 0 ? 0 : (wo_lo + d.stride_w - 1) / d.stride_w;
    const int64_t wo_hi = min(d.Wo - 1, wp / d.stride_w);
    float g = 0.f;
    for (int64_t ho = ho_lo; ho <= ho_hi; ++ho)
      for (int64_t wo = wo_lo; wo <= wo_hi; ++wo) {
        const int64_t o = ((n * d.Ho + ho) * d.Wo + wo) * d.C + c;
        if (nbk_load_as_f32(y, o, d.dtype) == xv) g += nbk_load_as_f32(dy, o, d.dtype);
      }
    nbk_store_from_f32(dx, i, d.dtype, g);
  }
}

// fp32 with a channel count that is a multiple of 4, 16-byte aligned tensors and fewer than 2^31
// elements: a lane takes four channels of a pixel (16-byte accesses) and the index arithmetic
// is 32-bit (the forms above divide 64-bit numbers five to seven times per element).  Same
// comparisons and the same order of additions, so the same results.
__global__ __launch_bounds__(256) void maxpool_fwd_vec4_kernel(const float4* __restrict__ x,
                                                               float4* __restrict__ y, nbk_pool_desc d) {
  const int C4 = (int)d.C >> 2, H = (int)d.H, W = (int)d.W, Ho = (int)d.Ho, Wo = (int)d.Wo;
  const int total = (int)(d.N * d.Ho * d.Wo) * C4;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    const int c = i % C4;
    int t = i / C4;
    const int wo = t % Wo; t /= Wo;
    const int ho = t % Ho;
    const int n = t / Ho;
    const int h0 = max(0, ho * d.stride_h - d.pad_t), h1 = min(H, ho * d.stride_h - d.pad_t + (int)d.kh);
    const int w0 = max(0, wo * d.stride_w - d.pad_l), w1 = min(W, wo * d.stride_w - d.pad_l + (int)d.kw);
    float4 m = make_float4(-INFINITY, -INFINITY, -INFINITY, -INFINITY);
    for (int h = h0; h < h1; ++h)
      for (int w = w0; w < w1; ++w) {
        const float4 v = x[((n * H + h) * W + w) * C4 + c];
        m.x = fmaxf(m.x, v.x); m.y = fmaxf(m.y, v.y); m.z = fmaxf(m.z, v.z); m.w = fmaxf(m.w, v.w);
      }
    y[i] = m;
  }
}

__global__ __launch_bounds__(256) void maxpool_bwd_vec4_kernel(const float4* __restrict__ x,
                                                               const float4* __restrict__ y,
                                                               const float4* __restrict__ dy,
                                                               float4* __restrict__ dx, nbk_pool_desc d) {
  const int C4 = (int)d.C >> 2, H = (int)d.H, W = (int)d.W, Ho = (int)d.Ho, Wo = (int)d.Wo;
  const int kh = (int)d.kh, kw = (int)d.kw;
  const int total = (int)(d.N * d.H * d.W) * C4;
  for (int i = blockIdx.x * 256 + threadIdx.x; i < total; i += gridDim.x * 256) {
    const int c = i % C4;
    int t = i / C4;
    const int w = t % W; t /= W;
    const int h = t % H;
    const int n = t / H;
    const float4 xv = x[i];
    const int hp = h + d.pad_t, wp = w + d.pad_l;
    int ho_lo = hp - kh + 1;
    ho_lo = ho_lo <= 0 ? 0 : (ho_lo + d.stride_h - 1) / d.stride_h;
    const int ho_hi = min(Ho - 1, hp / d.stride_h);
    int wo_lo = wp - kw + 1;
    wo_lo = wo_lo <= 0 ? 0 : (wo_lo + d.stride_w - 1) / d.stride_w;
    const int wo_hi = min(Wo - 1, wp / d.stride_w);
    float4 g = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int ho = ho_lo; ho <= ho_hi; ++ho)
      for (int wo = wo_lo; wo <= wo_hi; ++wo) {
        const int o = ((n * Ho + ho) * Wo + wo) * C4 + c;
        const float4 yv = y[o], gv = dy[o];
        if (yv.x == xv.x) g.x += gv.x;
        if (yv.y == xv.y) g.y += gv.y;
        if (yv.z == xv.z) g.z += gv.z;
        if (yv.w == xv.w) g.w += gv.w;
      }
    dx[i] = g;
  }
}

static bool pool_vec4_fits(const nbk_pool_desc* d, const void* p0, const void* p1, const void* p2,
                           const void* p3) {
  const uintptr_t bits = (uintptr_t)p0 | (uintptr_t)p1 | (uintptr_t)p2 | (uintptr_t)p3;
  return d->dtype == NBK_F32 && d->C % 4 == 0 && (bits & 15) == 0 &&
         d->N * d->H * d->W * d->C < 0x7fffffffLL && d->N * d->Ho * d->Wo * d->C < 0x7fffffffLL &&
         d->kh < (1 << 20) && d->kw < (1 << 20);
}

__global__ __launch_bounds__(256) void avgpool_fwd_kernel(const void* __restrict__ x,
                                                          void* __restrict__ y, nbk_pool_desc d) {
  const int64_t total = d.N * d.Ho * d.Wo * d.C;
  const float inv = 1.0f / (float)(d.kh * d.kw);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int64_t c = i % d.C;
    int64_t t = i / d.C;
    const int64_t wo = t % d.Wo; t /= d.Wo;
    const int64_t ho = t % d.Ho;
    const int64_t n = t / d.Ho;
    const int64_t h0 = max((int64_t)0, ho * d.stride_h - d.pad_t);
    const int64_t h1 = min(d.H, ho * d.stride_h - d.pad_t + d.kh);
    const int64_t w0 = max((int64_t)0, wo * d.stride_w - d.pad_l);
    const int64_t w1 = min(d.W, wo * d.stride_w - d.pad_l + d.kw);
    float s = 0.f;
    for (int64_t h = h0; h < h1; ++h)
      for (int64_t w = w0; w < w1; ++w)
        s += nbk_load_as_f32(x, ((n * d.H + h) * d.W + w) * d.C + c, d.dtype);
    nbk_store_from_f32(y, i, d.dtype, s * inv);
  }
}

__global__ __launch_bounds__(256) void avgpool_bwd_kernel(const void* __restrict__ dy,
                                                          void* __restrict__ dx, nbk_pool_desc d) {
  // gather form: each input element sums the cotangents of the windows that contain it
  const int64_t total = d.N * d.H * d.W * d.C;
  const float inv = 1.0f / (float)(d.kh * d.kw);
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total;
       i += (int64_t)gridDim.x * 256) {
    const int64_t c = i % d.C;
    int64_t t = i / d.C;
    const int64_t w = t % d.W; t /= d.W;
    const int64_t h = t % d.H;
    const int64_t n = t / d.H;
    const int64_t hp = h + d.pad_t, wp = w + d.pad_l;
    int64_t ho_lo = hp - d.kh + 1;
    ho_lo = ho_lo <= 0 ? 0 : (ho_lo + d.stride_h - 1) / d.stride_h;
    const int64_t ho_hi = min(d.Ho - 1, hp / d.stride_h);
    int64_t wo_lo = wp - d.kw + 1;
    wo_lo = wo_lo <= 0 ? 0 : (wo_lo + d.stride_w - 1) / d.stride_w;
    const int64_t wo_hi = min(d.Wo - 1, wp / d.stride_w);
    float g = 0.f;
    for (int64_t ho = ho_lo; ho <= ho_hi; ++ho)
      for (int64_t wo = wo_lo; wo <= wo_hi; ++wo)
        g += nbk_load_as_f32(dy, ((n * d.Ho + ho) * d.Wo + wo) * d.C + c, d.dtype);
    nbk_store_from_f32(dx, i, d.dtype, g * inv);
  }
}

static int pool_check(const nbk_pool_desc* d) {
  NBK_REQUIRE(d != nullptr, "pool: null descriptor");
  NBK_REQUIRE(d->N > 0 && d->H > 0 && d->W > 0 && d->C > 0 && d->Ho > 0 && d->Wo > 0,
              "pool: empty extent");
  NBK_REQUIRE(d->kh > 0 && d->kw > 0 && d->stride_h > 0 && d->stride_w > 0, "pool: bad window");
  NBK_REQUIRE(d->pad_t >= 0 && d->pad_l >= 0, "pool: negative padding");
  NBK_REQUIRE(d->dtype == NBK_F32 || d->dtype == NBK_BF16, "pool: dtype %d", d->dtype);
  return NBK_OK;
}

extern "C" int nbk_maxpool2d_fwd(const nbk_pool_desc* d, const void* x, void* y, void* stream) {
  int rc = pool_check(d);
  if (rc) return rc;
  NBK_REQUIRE(x && y, "pool: null pointer");
  int64_t total = d->N * d->Ho * d->Wo * d->C;
  if (pool_vec4_fits(d, x, y, nullptr, nullptr)) {
    int64_t vblocks = (total / 4 + 255) / 256;
    if (vblocks > 1 << 20) vblocks = 1 << 20;
    hipLaunchKernelGGL(maxpool_fwd_vec4_kernel, dim3((unsigned)vblocks), dim3(256), 0, (hipStream_t)stream,
                       (const float4*)x, (float4*)y, *d);
    return nbk_check_launch("maxpool_fwd_vec4_kernel");
  }
  int64_t blocks = (total + 255) / 256;
  if (blocks > 1 << 20) blocks = 1 << 20;
  hipLaunchKernelGGL(maxpool_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     x, y, *d);
  return nbk_check_launch("maxpool_fwd_kernel");
}

extern "C" int nbk_maxpool2d_bwd(const nbk_pool_desc* d, const void* x, const void* y,
                                 const void* dy, void* dx, void* stream) {
  int rc = pool_check(d);
  if (rc) return rc;
  NBK_REQUIRE(x && y && dy && dx, "pool: null pointer");
  int64_t total = d->N * d->H * d->W * d->C;
  if (pool_vec4_fits(d, x, y, dy, dx)) {
    int64_t vblocks = (total / 4 + 255) / 256;
    if (vblocks > 1 << 20) vblocks = 1 << 20;
    hipLaunchKernelGGL(maxpool_bwd_vec4_kernel, dim3((unsigned)vblocks), dim3(256), 0, (hipStream_t)stream,
                       (const float4*)x, (const float4*)y, (const float4*)dy, (float4*)dx, *d);
    return nbk_check_launch("maxpool_bwd_vec4_kernel");
  }
  int64_t blocks = (total + 255) / 256;
  if (blocks > 1 << 20) blocks = 1 << 20;
  hipLaunchKernelGGL(maxpool_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     x, y, dy, dx, *d);
  return nbk_check_launch("maxpool_bwd_kernel");
}

extern "C" int nbk_avgpool2d_fwd(const nbk_pool_desc* d, const void* x, void* y, void* stream) {
  int rc = pool_check(d);
  if (rc) return rc;
  NBK_REQUIRE(x && y, "pool: null pointer");
  int64_t total = d->N * d->Ho * d->Wo * d->C;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 1 << 20) blocks = 1 << 20;
  hipLaunchKernelGGL(avgpool_fwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     x, y, *d);
  return nbk_check_launch("avgpool_fwd_kernel");
}

extern "C" int nbk_avgpool2d_bwd(const nbk_pool_desc* d, const void* dy, void* dx, void* stream) {
  int rc = pool_check(d);
  if (rc) return rc;
  NBK_REQUIRE(dy && dx, "pool: null pointer");
  int64_t total = d->N * d->H * d->W * d->C;
  int64_t blocks = (total + 255) / 256;
  if (blocks > 1 << 20) blocks = 1 << 20;
  hipLaunchKernelGGL(avgpool_bwd_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     dy, dx, *d);
  return nbk_check_launch("avgpool_bwd_kernel");
}
