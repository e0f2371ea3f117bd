// conv2d (NHWC x RSCK) forward, input gradient and filter gradient as implicit
// GEMMs on v_mfma_f32_32x32x2f32.  No im2col buffer is materialised: the A / B
// tile loaders compute the gather addresses of each 128 x 16 / 16 x 128 tile.
//
//   forward : M = N*Ho*Wo   Ng = Cout   K = R*S*Cin
//             A[m,k] = x[n, ho*sh-pt+r, wo*sw-pl+s, c]      B[k,j] = w[r,s,c,j]
//   dgrad   : M = N*H*W     Ng = Cin    K = R*S*Cout
//             A[m,k] = dy[n, (h+pt-r)/sh, (w+pl-s)/sw, co]  B[k,j] = w[r,s,j,co]
//   wgrad   : M = R*S*Cin   Ng = Cout   K = N*Ho*Wo
//             A[m,k] = x[n, ho*sh-pt+r, wo*sw-pl+s, c]      B[k,j] = dy[n,ho,wo,j]
// Out-of-image taps read zero, which is the zero padding of the reference op.
#include "nbk_common.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { CONV_FWD = 0, CONV_DGRAD = 1, CONV_WGRAD = 2 };

struct ConvArgs {
  nbk_conv_desc d;
  const float* a;     // x (fwd, wgrad) or dy (dgrad)
  const float* b;     // w (fwd, dgrad) or dy (wgrad)
  const float* bias;  // fwd only
  float* out;
  int64_t M, Ng, K;
  int32_t tiles_m, tiles_n;
};

template <int MODE>
__device__ __forceinline__ float conv_load_a(const ConvArgs& g, int64_t m, int64_t k) {
  const nbk_conv_desc& d = g.d;
  if (m >= g.M || k >= g.K) return 0.f;
  if (MODE == CONV_FWD) {
    const int64_t c = k % d.Cin;
    const int64_t rs = k / d.Cin;
    const int64_t s = rs % d.S, r = rs / d.S;
    const int64_t wo = m % d.Wo;
    const int64_t t = m / d.Wo;
    const int64_t ho = t % d.Ho, n = t / d.Ho;
    const int64_t h = ho * d.stride_h - d.pad_t + r, w = wo * d.stride_w - d.pad_l + s;
    if (h < 0 || h >= d.H || w < 0 || w >= d.W) return 0.f;
    return g.a[((n * d.H + h) * d.W + w) * d.Cin + c];
  } else if (MODE == CONV_DGRAD) {
    const int64_t co = k % d.Cout;
    const int64_t rs = k / d.Cout;
    const int64_t s = rs % d.S, r = rs / d.S;
    const int64_t w = m % d.W;
    const int64_t t = m / d.W;
    const int64_t h = t % d.H, n = t / d.H;
    const int64_t hn = h + d.pad_t - r, wn = w + d.pad_l - s;
    if (hn < 0 || wn < 0 || hn % d.stride_h != 0 || wn % d.stride_w != 0) return 0.f;
    const int64_t ho = hn / d.stride_h, wo = wn / d.stride_w;
    if (ho >= d.Ho || wo >= d.Wo) return 0.f;
    return g.a[((n * d.Ho + ho) * d.Wo + wo) * d.Cout + co];
  } else {
    const int64_t c = m % d.Cin;
    const int64_t rs = m / d.Cin;
    const int64_t s = rs % d.S, r = rs / d.S;
    const int64_t wo = k % d.Wo;
    const int64_t t = k / d.Wo;
    const int64_t ho = t % d.Ho, n = t / d.Ho;
    const int64_t h = ho * d.stride_h - d.pad_t + r, w = wo * d.stride_w - d.pad_l + s;
    if (h < 0 || h >= d.H || w < 0 || w >= d.W) return 0.f;
    return g.a[((n * d.H + h) * d.W + w) * d.Cin + c];
  }
}

template <int MODE>
__device__ __forceinline__ float conv_load_b(const ConvArgs& g, int64_t k, int64_t j) {
  const nbk_conv_desc& d = g.d;
  if (k >= g.K || j >= g.Ng) return 0.f;
  if (MODE == CONV_FWD) return g.b[k * d.Cout + j];  // w viewed as [R*S*Cin, Cout]
  if (MODE == CONV_DGRAD) {
    const int64_t co = k % d.Cout, rs = k / d.Cout;
    return g.b[(rs * d.Cin + j) * d.Cout + co];
  }
  return g.b[k * d.Cout + j];  // dy viewed as [N*Ho*Wo, Cout]
}

template <int MODE>
__global__ __launch_bounds__(256) void conv_kernel(const ConvArgs g) {
  constexpr int BK = 16, LD = 128 + 4;
  __shared__ float As[2][BK][LD];
  __shared__ float Bs[2][BK][LD];
  const int tm_i = blockIdx.x % g.tiles_m, tn_i = blockIdx.x / g.tiles_m;
  const int64_t m0 = (int64_t)tm_i * 128, n0 = (int64_t)tn_i * 128;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 64;
  const int li = lane & 31, kg = lane >> 5;

  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) acc[i][j] = (f32x16)(0.f);

  // A staging: forward / dgrad walk k fastest (channels are contiguous in
  // memory), wgrad walks m fastest.  B is always contiguous along j.
  float ra[8], rb[8];
  auto load_a = [&](int64_t k0) {
    if (MODE == CONV_WGRAD) {
      const int kk = tid >> 4, rr = (tid & 15) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) ra[e] = conv_load_a<MODE>(g, m0 + rr + e, k0 + kk);
    } else {
      const int row = tid >> 1, kk = (tid & 1) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) ra[e] = conv_load_a<MODE>(g, m0 + row, k0 + kk + e);
    }
  };
  auto store_a = [&](float (*S)[LD]) {
    if (MODE == CONV_WGRAD) {
      const int kk = tid >> 4, rr = (tid & 15) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) S[kk][rr + e] = ra[e];
    } else {
      const int row = tid >> 1, kk = (tid & 1) * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) S[kk + e][row] = ra[e];
    }
  };
  auto load_b = [&](int64_t k0) {
    const int kk = tid >> 4, jj = (tid & 15) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) rb[e] = conv_load_b<MODE>(g, k0 + kk, n0 + jj + e);
  };
  auto store_b = [&](float (*S)[LD]) {
    const int kk = tid >> 4, jj = (tid & 15) * 8;
#pragma unroll
    for (int e = 0; e < 8; ++e) S[kk][jj + e] = rb[e];
  };

  const int64_t nk = (g.K + BK - 1) / BK;
  load_a(0);
  load_b(0);
  store_a(As[0]);
  store_b(Bs[0]);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      load_a((kt + 1) * BK);
      load_b((kt + 1) * BK);
    }
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
      const int k = ks * 2 + kg;
      float fa[2], fb[2];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = As[cur][k][wm + i * 32 + li];
#pragma unroll
      for (int j = 0; j < 2; ++j) fb[j] = Bs[cur][k][wn + j * 32 + li];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
    }
    if (more) {
      store_a(As[cur ^ 1]);
      store_b(Bs[cur ^ 1]);
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int64_t col = n0 + wn + j * 32 + li;
      const bool col_ok = col < g.Ng;
      const float bv = (g.bias && col_ok) ? g.bias[col] : 0.f;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm + i * 32 + (r >> 2) * 8 + kg * 4 + (r & 3);
        if (col_ok && row < g.M) g.out[row * g.Ng + col] = acc[i][j][r] + bv;
      }
    }
}

static int conv_check(const nbk_conv_desc* d) {
  NBK_REQUIRE(d != nullptr, "conv2d: null descriptor");
  NBK_REQUIRE(d->dtype == NBK_F32, "conv2d: only fp32 is implemented (dtype %d)", d->dtype);
  NBK_REQUIRE(d->N > 0 && d->H > 0 && d->W > 0 && d->Cin > 0 && d->R > 0 && d->S > 0 &&
                  d->Cout > 0 && d->Ho > 0 && d->Wo > 0,
              "conv2d: empty extent");
  NBK_REQUIRE(d->stride_h > 0 && d->stride_w > 0, "stride values must be > 0");
  NBK_REQUIRE(d->pad_t >= 0 && d->pad_b >= 0 && d->pad_l >= 0 && d->pad_r >= 0,
              "padding values must be >= 0");
  const int64_t ho = (d->H + d->pad_t + d->pad_b - d->R) / d->stride_h + 1;
  const int64_t wo = (d->W + d->pad_l + d->pad_r - d->S) / d->stride_w + 1;
  NBK_REQUIRE(ho == d->Ho && wo == d->Wo, "conv2d: output size %lld x %lld does not match %lld x %lld",
              (long long)d->Ho, (long long)d->Wo, (long long)ho, (long long)wo);
  return NBK_OK;
}

template <int MODE>
static int conv_launch(ConvArgs& a, hipStream_t st) {
  a.tiles_m = (int)((a.M + 127) / 128);
  a.tiles_n = (int)((a.Ng + 127) / 128);
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n;
  NBK_REQUIRE(blocks <= 0x7fffffffLL, "conv2d: launch too large");
  hipLaunchKernelGGL(conv_kernel<MODE>, dim3((unsigned)blocks), dim3(256), 0, st, a);
  return nbk_check_launch("conv_kernel");
}

extern "C" int nbk_conv2d_fwd(const nbk_conv_desc* d, const void* x, const void* w,
                              const void* bias, void* y, void* stream) {
  int rc = conv_check(d);
  if (rc) return rc;
  NBK_REQUIRE(x && w && y, "conv2d: null pointer");
  ConvArgs a;
  a.d = *d;
  a.a = (const float*)x; a.b = (const float*)w; a.bias = (const float*)bias; a.out = (float*)y;
  a.M = d->N * d->Ho * d->Wo; a.Ng = d->Cout; a.K = d->R * d->S * d->Cin;
  return conv_launch<CONV_FWD>(a, (hipStream_t)stream);
}

extern "C" int nbk_conv2d_dgrad(const nbk_conv_desc* d, const void* dy, const void* w, void* dx,
                                void* stream) {
  int rc = conv_check(d);
  if (rc) return rc;
  NBK_REQUIRE(dy && w && dx, "conv2d: null pointer");
  ConvArgs a;
  a.d = *d;
  a.a = (const float*)dy; a.b = (const float*)w; a.bias = nullptr; a.out = (float*)dx;
  a.M = d->N * d->H * d->W; a.Ng = d->Cin; a.K = d->R * d->S * d->Cout;
  return conv_launch<CONV_DGRAD>(a, (hipStream_t)stream);
}

extern "C" int nbk_conv2d_wgrad(const nbk_conv_desc* d, const void* x, const void* dy, void* dw,
                                void* stream) {
  int rc = conv_check(d);
  if (rc) return rc;
  NBK_REQUIRE(x && dy && dw, "conv2d: null pointer");
  ConvArgs a;
  a.d = *d;
  a.a = (const float*)x; a.b = (const float*)dy; a.bias = nullptr; a.out = (float*)dw;
  a.M = d->R * d->S * d->Cin; a.Ng = d->Cout; a.K = d->N * d->Ho * d->Wo;
  return conv_launch<CONV_WGRAD>(a, (hipStream_t)stream);
}
