// conv2d (NHWC x RSCK) forward, input gradient and filter gradient as implicit
// GEMMs on v_mfma_f32_32x32x2f32.  No im2col buffer is materialised: the tile
// loaders gather straight from the image.
//
//   forward : M = N*Ho*Wo   Ng = Cout   K = R*S*Cin   (k = (r, s, c), c fastest)
//             A[m,k] = x[n, ho*sh-pt+r, wo*sw-pl+s, c]      B[k,j] = w[r,s,c,j]
//   dgrad   : M = N*H*W     Ng = Cin    K = R*S*Cout  (k = (r, s, co))
//             A[m,k] = dy[n, (h+pt-r)/sh, (w+pl-s)/sw, co]  B[k,j] = w[r,s,j,co]
//   wgrad   : M = R*S*Cin   Ng = Cout   K = N*Ho*Wo   (k = output pixel)
//             A[m,k] = x[n, ho*sh-pt+r, wo*sw-pl+s, c]      B[k,j] = dy[n,ho,wo,j]
// Out-of-image taps read zero, which is the zero padding of the reference op.
//
// Address arithmetic is kept out of the K loop: a lane owns one output pixel
// (forward, dgrad) or one run of 8 filter rows (wgrad) for the whole tile and
// decomposes it once; with channel counts that are multiples of 16 (8 for wgrad)
// a 16-wide K step lies inside one filter tap, the tap is uniform across the
// workgroup, and every lane fetches 8 consecutive channels as two 16-byte loads
// (FAST).  Other channel counts take the element-wise gather.
// wgrad contracts over every output pixel of the batch while its result is tiny,
// so it is split along K over blockIdx.z into a workspace and summed by a second
// kernel in a fixed order (no atomics: results do not depend on scheduling).
#include "nbk_common.h"

typedef float f32x16 __attribute__((ext_vector_type(16)));

enum { CONV_FWD = 0, CONV_DGRAD = 1, CONV_WGRAD = 2 };

// Division of a number below 2^31 by a divisor fixed for the launch as a multiplication: the
// host finds mul = ceil(2^(31 + shift) / d) with shift = ceil(log2 d), which fits 32 bits, and
// n / d = (n * mul) >> (31 + shift) exactly for 0 <= n < 2^31 (five instructions where the
// division takes twenty-odd).
struct ConvDiv {
  uint32_t mul, shift, d, pad;
  __host__ void set(int64_t div) {
    d = (uint32_t)div;
    shift = 0;
    while ((1ull << shift) < (uint64_t)div) ++shift;
    mul = (uint32_t)(((1ull << (31 + shift)) + (uint64_t)div - 1) / (uint64_t)div);
  }
  __device__ __forceinline__ int quot(int n) const {
    return (int)(((uint64_t)(uint32_t)n * mul) >> (31 + shift));
  }
  // quotient and remainder of n >= 0
  __device__ __forceinline__ int divmod(int n, int& rem) const {
    const int q = quot(n);
    rem = n - q * (int)d;
    return q;
  }
};

struct ConvArgs {
  nbk_conv_desc d;
  const float* a;     // x (fwd, wgrad) or dy (dgrad)
  const float* b;     // w (fwd, dgrad) or dy (wgrad)
  const float* bias;  // fwd only
  float* out;         // result, or the [splits, M, Ng] workspace when splits > 1
  int64_t M, Ng, K;
  int64_t k_per_split;  // multiple of 16
  int32_t tiles_m, tiles_n, splits;
  ConvDiv by_cin, by_cout, by_s, by_w, by_h, by_wo, by_ho;
  __host__ void set_divisors() {
    by_cin.set(d.Cin); by_cout.set(d.Cout); by_s.set(d.S);
    by_w.set(d.W); by_h.set(d.H); by_wo.set(d.Wo); by_ho.set(d.Ho);
  }
};

// ---- element-wise gather (any channel count) ----------------------------------------------
// (every extent that is divided here fits 32 bits, checked on the host: 64-bit divisions would
// cost ten times the instructions, eight times per element)
template <int MODE>
__device__ __forceinline__ float conv_load_a(const ConvArgs& g, int64_t m64, int64_t k64, int64_t k_end) {
  const nbk_conv_desc& d = g.d;
  if (m64 >= g.M || k64 >= k_end) return 0.f;
  const int m = (int)m64, k = (int)k64;
  const int Cin = (int)d.Cin, Cout = (int)d.Cout, S = (int)d.S, H = (int)d.H, W = (int)d.W,
            Ho = (int)d.Ho, Wo = (int)d.Wo;
  if (MODE == CONV_FWD) {
    int c, s, wo, ho;
    const int rs = g.by_cin.divmod(k, c);
    const int r = g.by_s.divmod(rs, s);
    const int t = g.by_wo.divmod(m, wo);
    const int n = g.by_ho.divmod(t, ho);
    const int h = ho * d.stride_h - d.pad_t + r, w = wo * d.stride_w - d.pad_l + s;
    if (h < 0 || h >= H || w < 0 || w >= W) return 0.f;
    return g.a[(int64_t)((n * H + h) * W + w) * Cin + c];
  } else if (MODE == CONV_DGRAD) {
    int co, s, w, h;
    const int rs = g.by_cout.divmod(k, co);
    const int r = g.by_s.divmod(rs, s);
    const int t = g.by_w.divmod(m, w);
    const int n = g.by_h.divmod(t, h);
    const int hn = h + d.pad_t - r, wn = w + d.pad_l - s;
    if (hn < 0 || wn < 0 || hn % d.stride_h != 0 || wn % d.stride_w != 0) return 0.f;
    const int ho = hn / d.stride_h, wo = wn / d.stride_w;
    if (ho >= Ho || wo >= Wo) return 0.f;
    return g.a[(int64_t)((n * Ho + ho) * Wo + wo) * Cout + co];
  } else {
    int c, s, wo, ho;
    const int rs = g.by_cin.divmod(m, c);
    const int r = g.by_s.divmod(rs, s);
    const int t = g.by_wo.divmod(k, wo);
    const int n = g.by_ho.divmod(t, ho);
    const int h = ho * d.stride_h - d.pad_t + r, w = wo * d.stride_w - d.pad_l + s;
    if (h < 0 || h >= H || w < 0 || w >= W) return 0.f;
    return g.a[(int64_t)((n * H + h) * W + w) * Cin + c];
  }
}

template <int MODE>
__device__ __forceinline__ float conv_load_b(const ConvArgs& g, int64_t k, int64_t j, int64_t k_end) {
  const nbk_conv_desc& d = g.d;
  if (k >= k_end || j >= g.Ng) return 0.f;
  if (MODE == CONV_FWD) return g.b[k * d.Cout + j];  // w viewed as [R*S*Cin, Cout]
  if (MODE == CONV_DGRAD) {
    int co;
    const int rs = g.by_cout.divmod((int)k, co);
    return g.b[((int64_t)rs * d.Cin + j) * d.Cout + co];
  }
  return g.b[k * d.Cout + j];  // dy viewed as [N*Ho*Wo, Cout]
}

__device__ __forceinline__ void conv_ld8(const float* p, bool ok, float* r) {
  float4 v0 = make_float4(0.f, 0.f, 0.f, 0.f), v1 = v0;
  if (ok) {
    v0 = *(const float4*)p;
    v1 = *(const float4*)(p + 4);
  }
  r[0] = v0.x; r[1] = v0.y; r[2] = v0.z; r[3] = v0.w;
  r[4] = v1.x; r[5] = v1.y; r[6] = v1.z; r[7] = v1.w;
}

// NJ: 32-column MFMA tiles per wave along the output's channel axis: 2 for a 128 x 128
// workgroup tile, 1 for 128 x 64 (channel counts up to 64 would waste half of the wider tile).
template <int MODE, bool FAST, int NJ>
__global__ __launch_bounds__(256) void conv_kernel(const ConvArgs g) {
  // Tiles sit in LDS k-major, [k][128 rows], with the rows of k-row k rotated by 32 places when
  // (k ^ k / 8) is odd.  The two halves of a wave read k-rows 2 ks and 2 ks + 1 of one MFMA
  // step, and the two lanes of a pixel store k-rows e and 8 + e: either way the halves land
  // 32 banks apart (a padded pitch of 132 serves the stores only: 77-87 % of the LDS cycles of
  // these kernels were bank conflicts).
  constexpr int BK = 16, LD = 128, BN = 64 * NJ;
  __shared__ float As[2][BK][LD];
  __shared__ float Bs[2][BK][LD];
  auto rot = [](int k, int col) { return (col + 32 * ((k ^ (k >> 3)) & 1)) & 127; };
  const nbk_conv_desc& d = g.d;
  const int tm_i = blockIdx.x % g.tiles_m, tn_i = blockIdx.x / g.tiles_m;
  const int64_t m0 = (int64_t)tm_i * 128, n0 = (int64_t)tn_i * BN;
  const int64_t k_begin = (int64_t)blockIdx.z * g.k_per_split;
  const int64_t k_end = min(g.K, k_begin + g.k_per_split);
  float* out = g.out + (g.splits > 1 ? (int64_t)blockIdx.z * g.M * g.Ng : 0);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = (wave >> 1) * 64, wn = (wave & 1) * 32 * NJ;
  const int li = lane & 31, kg = lane >> 5;

  f32x16 acc[2][NJ];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < NJ; ++j) acc[i][j] = (f32x16)(0.f);

  // ---- per-lane constants of the A gather ----
  // forward / dgrad: the lane's pixel; wgrad: the lane's first filter row and, as running
  // state, the pixel of its K column.
  const int a_row = tid >> 1, a_kk = (tid & 1) * 8;  // fwd / dgrad: pixel row, 8 k
  const int w_kk = tid >> 4, w_rr = (tid & 15) * 8;  // wgrad: pixel column, 8 filter rows
  int p_n = 0, p_y = 0, p_x = 0;
  bool p_ok = false;
  int f_r = 0, f_s = 0, f_c = 0;
  bool f_ok = false;
  if (MODE == CONV_WGRAD) {
    const int64_t m = m0 + w_rr;
    f_ok = m < g.M;
    const int mm = f_ok ? (int)m : 0;
    f_c = mm % (int)d.Cin;
    const int rs = mm / (int)d.Cin;
    f_s = rs % (int)d.S;
    f_r = rs / (int)d.S;
    const int64_t px = k_begin + w_kk;  // < 2^31 (checked on the host)
    p_x = (int)(px % d.Wo);
    const int t = (int)(px / d.Wo);
    p_y = t % (int)d.Ho;
    p_n = t / (int)d.Ho;
  } else {
    const int64_t m = m0 + a_row;
    p_ok = m < g.M;
    const int mm = p_ok ? (int)m : 0;
    const int wd = MODE == CONV_FWD ? (int)d.Wo : (int)d.W;
    const int hd = MODE == CONV_FWD ? (int)d.Ho : (int)d.H;
    p_x = mm % wd;
    const int t = mm / wd;
    p_y = t % hd;
    p_n = t / hd;
  }

  float ra[8], rb[8];
  const bool unit_stride = d.stride_h == 1 && d.stride_w == 1;
  // forward / dgrad, FAST: the filter tap (t_r, t_s) and the first channel t_c of the K step
  // that is loaded next (uniform; kept as running counters: a 64-bit division per K step and
  // operand otherwise)
  int t_r = 0, t_s = 0, t_c = 0;
  if (FAST && MODE != CONV_WGRAD) {
    const int ck = MODE == CONV_FWD ? (int)d.Cin : (int)d.Cout;
    const int tap = (int)(k_begin / ck);
    t_c = (int)(k_begin - (int64_t)tap * ck);
    t_r = tap / (int)d.S;
    t_s = tap - t_r * (int)d.S;
  }
  // forward: row, column and number of the lane's input pixel at tap (0, 0); dgrad with unit
  // stride: the same for its output pixel
  int q_h0 = 0, q_w0 = 0, q_pix0 = 0;
  if (MODE == CONV_FWD) {
    q_h0 = p_y * d.stride_h - d.pad_t;
    q_w0 = p_x * d.stride_w - d.pad_l;
    q_pix0 = (p_n * (int)d.H + q_h0) * (int)d.W + q_w0;
  } else if (MODE == CONV_DGRAD) {
    q_h0 = p_y + d.pad_t;
    q_w0 = p_x + d.pad_l;
    q_pix0 = (p_n * (int)d.Ho + q_h0) * (int)d.Wo + q_w0;
  }
  auto next_tap = [&]() {
    if (FAST && MODE != CONV_WGRAD) {
      const int ck = MODE == CONV_FWD ? (int)d.Cin : (int)d.Cout;
      t_c += BK;
      if (t_c >= ck) {
        t_c -= ck;
        if (++t_s == (int)d.S) { t_s = 0; ++t_r; }
      }
    }
  };
  auto load_a = [&](int64_t k0) {
    if (MODE == CONV_WGRAD) {
      // pixel (p_n, p_y, p_x) is column k0 + w_kk; taps of rows m0 + w_rr .. + 7
      const bool k_ok = k0 + w_kk < k_end;
      if (FAST) {
        const int h = p_y * d.stride_h - d.pad_t + f_r, w = p_x * d.stride_w - d.pad_l + f_s;
        const bool ok = f_ok && k_ok && h >= 0 && h < d.H && w >= 0 && w < d.W;
        conv_ld8(g.a + (((int64_t)p_n * d.H + h) * d.W + w) * d.Cin + f_c, ok, ra);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) ra[e] = conv_load_a<MODE>(g, m0 + w_rr + e, k0 + w_kk, k_end);
      }
      // advance the pixel by one K step
      p_x += BK;
      while (p_x >= d.Wo) {
        p_x -= (int)d.Wo;
        if (++p_y >= d.Ho) { p_y = 0; ++p_n; }
      }
    } else if (FAST) {
      const int c0 = t_c + a_kk, r = t_r, s = t_s;
      if (MODE == CONV_FWD) {
        // (the lane's pixel at tap (0, 0) is a constant of the lane; the tap adds a uniform
        // number of pixels; pixel numbers fit 32 bits, checked on the host)
        const int h = q_h0 + r, w = q_w0 + s;
        const bool ok = p_ok && h >= 0 && h < d.H && w >= 0 && w < d.W;
        conv_ld8(g.a + (int64_t)(q_pix0 + r * (int)d.W + s) * d.Cin + c0, ok, ra);
      } else if (unit_stride) {
        const int ho = q_h0 - r, wo = q_w0 - s;
        const bool ok = p_ok && ho >= 0 && wo >= 0 && ho < d.Ho && wo < d.Wo;
        conv_ld8(g.a + (int64_t)(q_pix0 - r * (int)d.Wo - s) * d.Cout + c0, ok, ra);
      } else {  // (two integer divisions per lane and K step)
        const int hn = p_y + d.pad_t - r, wn = p_x + d.pad_l - s;
        const int ho = hn / d.stride_h, wo = wn / d.stride_w;
        const bool ok = p_ok && hn >= 0 && wn >= 0 && ho * d.stride_h == hn &&
                        wo * d.stride_w == wn && ho < d.Ho && wo < d.Wo;
        conv_ld8(g.a + (((int64_t)p_n * d.Ho + ho) * d.Wo + wo) * d.Cout + c0, ok, ra);
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) ra[e] = conv_load_a<MODE>(g, m0 + a_row, k0 + a_kk + e, k_end);
    }
  };
  auto store_a = [&](float (*S)[LD]) {
    if (MODE == CONV_WGRAD) {
#pragma unroll
      for (int e = 0; e < 8; ++e) S[w_kk][rot(w_kk, w_rr) + e] = ra[e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) S[a_kk + e][rot(a_kk + e, a_row)] = ra[e];
    }
  };
  auto load_b = [&](int64_t k0) {
    if (MODE == CONV_DGRAD) {
      // w[r, s, j, co]: contiguous along k = co for a fixed input channel j
      const int64_t j = n0 + a_row;
      if (FAST) {
        const int tap = t_r * (int)d.S + t_s, co = t_c + a_kk;
        conv_ld8(g.b + ((int64_t)tap * d.Cin + j) * d.Cout + co, j < g.Ng, rb);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) rb[e] = conv_load_b<MODE>(g, k0 + a_kk + e, j, k_end);
      }
    } else {
      // [K, Cout] row-major: w for the forward product, dy for wgrad
      const int64_t k = k0 + w_kk, j = n0 + w_rr;
      if (FAST) {
        conv_ld8(g.b + k * d.Cout + j, k < k_end && j < g.Ng, rb);
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) rb[e] = conv_load_b<MODE>(g, k, j + e, k_end);
      }
    }
  };
  auto store_b = [&](float (*S)[LD]) {
    if (MODE == CONV_DGRAD) {
#pragma unroll
      for (int e = 0; e < 8; ++e) S[a_kk + e][rot(a_kk + e, a_row)] = rb[e];
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) S[w_kk][rot(w_kk, w_rr) + e] = rb[e];
    }
  };

  const int64_t nk = (k_end - k_begin + BK - 1) / BK;
  load_a(k_begin);
  load_b(k_begin);
  next_tap();
  store_a(As[0]);
  store_b(Bs[0]);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    const bool more = kt + 1 < nk;
    if (more) {
      load_a(k_begin + (kt + 1) * BK);
      load_b(k_begin + (kt + 1) * BK);
      next_tap();
    }
#pragma unroll
    for (int ks = 0; ks < BK / 2; ++ks) {
      const int k = ks * 2 + kg;
      float fa[2], fb[NJ];
#pragma unroll
      for (int i = 0; i < 2; ++i) fa[i] = As[cur][k][rot(k, wm + i * 32 + li)];
#pragma unroll
      for (int j = 0; j < NJ; ++j) fb[j] = Bs[cur][k][rot(k, wn + j * 32 + li)];
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j)
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
    for (int j = 0; j < NJ; ++j) {
      const int64_t col = n0 + wn + j * 32 + li;
      const bool col_ok = col < g.Ng;
      const float bv = (g.bias && col_ok) ? g.bias[col] : 0.f;
      const bool relu = MODE == CONV_FWD && d.act == NBK_ACT_RELU;
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int64_t row = m0 + wm + i * 32 + (r >> 2) * 8 + kg * 4 + (r & 3);
        const float v = acc[i][j][r] + bv;
        if (col_ok && row < g.M) out[row * g.Ng + col] = relu ? fmaxf(v, 0.f) : v;
      }
    }
}

// out[i] = sum over z of partial[z][i]; eight slices are in flight per lane and the order
// of the additions is fixed, so the result does not depend on scheduling.
__global__ __launch_bounds__(256) void conv_sum_partials(const float* partial, float* out,
                                                         int64_t n, int splits) {
  for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256) {
    float s = 0.f;
    int z = 0;
    for (; z + 8 <= splits; z += 8) {
      float v[8];
#pragma unroll
      for (int q = 0; q < 8; ++q) v[q] = partial[(int64_t)(z + q) * n + i];
      s += ((v[0] + v[1]) + (v[2] + v[3])) + ((v[4] + v[5]) + (v[6] + v[7]));
    }
    for (; z < splits; ++z) s += partial[(int64_t)z * n + i];
    out[i] = s;
  }
}

static int conv_check(const nbk_conv_desc* d) {
  NBK_REQUIRE(d != nullptr, "conv2d: null descriptor");
  NBK_REQUIRE(d->dtype == NBK_F32, "conv2d: only fp32 is implemented (dtype %d)", d->dtype);
  NBK_REQUIRE(d->N > 0 && d->H > 0 && d->W > 0 && d->Cin > 0 && d->R > 0 && d->S > 0 &&
                  d->Cout > 0 && d->Ho > 0 && d->Wo > 0,
              "conv2d: empty extent");
  NBK_REQUIRE(d->act == NBK_ACT_NONE || d->act == NBK_ACT_RELU, "conv2d: act %d", d->act);
  NBK_REQUIRE(d->stride_h > 0 && d->stride_w > 0, "stride values must be > 0");
  NBK_REQUIRE(d->pad_t >= 0 && d->pad_b >= 0 && d->pad_l >= 0 && d->pad_r >= 0,
              "padding values must be >= 0");
  const int64_t ho = (d->H + d->pad_t + d->pad_b - d->R) / d->stride_h + 1;
  const int64_t wo = (d->W + d->pad_l + d->pad_r - d->S) / d->stride_w + 1;
  NBK_REQUIRE(ho == d->Ho && wo == d->Wo, "conv2d: output size %lld x %lld does not match %lld x %lld",
              (long long)d->Ho, (long long)d->Wo, (long long)ho, (long long)wo);
  NBK_REQUIRE(d->N * d->H * d->W < 0x7fffffffLL && d->N * d->Ho * d->Wo < 0x7fffffffLL &&
                  d->R * d->S * d->Cin < 0x7fffffffLL && d->R * d->S * d->Cout < 0x7fffffffLL,
              "conv2d: extent beyond 2^31 elements");
  return NBK_OK;
}

static bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

template <int MODE>
static int conv_launch(ConvArgs& a, bool fast, hipStream_t st) {
  // the narrow workgroup tile when the last 128-wide column tile would be at most half full,
  // or when the wide tiling gives fewer workgroups than the GPU has CUs
  a.set_divisors();
  const int64_t wide = ((a.M + 127) / 128) * ((a.Ng + 127) / 128) * a.splits;
  const bool narrow = (a.Ng - 1) % 128 < 64 || wide < nbk_num_cus();
  const int bn = narrow ? 64 : 128;
  a.tiles_m = (int)((a.M + 127) / 128);
  a.tiles_n = (int)((a.Ng + bn - 1) / bn);
  const int64_t blocks = (int64_t)a.tiles_m * a.tiles_n;
  NBK_REQUIRE(blocks <= 0x7fffffffLL, "conv2d: launch too large");
  const dim3 grid((unsigned)blocks, 1, (unsigned)a.splits);
  if (fast && narrow) hipLaunchKernelGGL((conv_kernel<MODE, true, 1>), grid, dim3(256), 0, st, a);
  else if (fast) hipLaunchKernelGGL((conv_kernel<MODE, true, 2>), grid, dim3(256), 0, st, a);
  else if (narrow) hipLaunchKernelGGL((conv_kernel<MODE, false, 1>), grid, dim3(256), 0, st, a);
  else hipLaunchKernelGGL((conv_kernel<MODE, false, 2>), grid, dim3(256), 0, st, a);
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
  a.splits = 1; a.k_per_split = (a.K + 15) / 16 * 16;
  const bool fast = d->Cin % 16 == 0 && d->Cout % 8 == 0 && aligned16(x) && aligned16(w);
  return conv_launch<CONV_FWD>(a, fast, (hipStream_t)stream);
}

extern "C" int nbk_conv2d_dgrad(const nbk_conv_desc* d, const void* dy, const void* w, void* dx,
                                void* stream) {
  int rc = conv_check(d);
  if (rc) return rc;
  NBK_REQUIRE(dy && w && dx, "conv2d: null pointer");
  NBK_REQUIRE(d->act == NBK_ACT_NONE, "conv2d: an activation goes with the forward product only");
  ConvArgs a;
  a.d = *d;
  a.a = (const float*)dy; a.b = (const float*)w; a.bias = nullptr; a.out = (float*)dx;
  a.M = d->N * d->H * d->W; a.Ng = d->Cin; a.K = d->R * d->S * d->Cout;
  a.splits = 1; a.k_per_split = (a.K + 15) / 16 * 16;
  const bool fast = d->Cout % 16 == 0 && aligned16(dy) && aligned16(w);
  return conv_launch<CONV_DGRAD>(a, fast, (hipStream_t)stream);
}

// K split of the filter-gradient product: as many workgroups as the GPU holds at once (two per
// CU) and no more -- a handful beyond that would run as a second round behind the first and
// nearly double the launch (515 workgroups for 512 places: 129 us, 500: 90) --, at least four
// K steps each.
static void wgrad_split(const nbk_conv_desc* d, int* splits, int64_t* k_per_split) {
  const int64_t M = d->R * d->S * d->Cin, K = d->N * d->Ho * d->Wo;
  const int64_t tiles = ((M + 127) / 128) * ((d->Cout + 127) / 128);
  int64_t want = 2 * (int64_t)nbk_num_cus() / tiles;
  const int64_t most = K / 64 > 0 ? K / 64 : 1;
  if (want > most) want = most;
  if (want < 1) want = 1;
  int64_t kps = (K + want - 1) / want;
  kps = (kps + 15) / 16 * 16;
  *k_per_split = kps;
  *splits = (int)((K + kps - 1) / kps);
}

extern "C" int64_t nbk_conv2d_wgrad_workspace(const nbk_conv_desc* d) {
  if (conv_check(d) != NBK_OK) return -1;
  int splits;
  int64_t kps;
  wgrad_split(d, &splits, &kps);
  if (splits <= 1) return 0;
  return (int64_t)splits * d->R * d->S * d->Cin * d->Cout * (int64_t)sizeof(float);
}

extern "C" int nbk_conv2d_wgrad(const nbk_conv_desc* d, const void* x, const void* dy, void* dw,
                                void* workspace, int64_t workspace_bytes, void* stream) {
  int rc = conv_check(d);
  if (rc) return rc;
  NBK_REQUIRE(x && dy && dw, "conv2d: null pointer");
  NBK_REQUIRE(d->act == NBK_ACT_NONE, "conv2d: an activation goes with the forward product only");
  ConvArgs a;
  a.d = *d;
  a.a = (const float*)x; a.b = (const float*)dy; a.bias = nullptr; a.out = (float*)dw;
  a.M = d->R * d->S * d->Cin; a.Ng = d->Cout; a.K = d->N * d->Ho * d->Wo;
  int splits;
  int64_t kps;
  wgrad_split(d, &splits, &kps);
  const int64_t need = (int64_t)splits * a.M * a.Ng * (int64_t)sizeof(float);
  if (splits > 1 && (workspace == nullptr || workspace_bytes < need || !aligned16(workspace))) {
    splits = 1;  // no room for partial sums: one pass over all of K
    kps = (a.K + 15) / 16 * 16;
  }
  a.splits = splits;
  a.k_per_split = kps;
  if (splits > 1) a.out = (float*)workspace;
  const bool fast = d->Cin % 8 == 0 && d->Cout % 8 == 0 && aligned16(x) && aligned16(dy);
  rc = conv_launch<CONV_WGRAD>(a, fast, (hipStream_t)stream);
  if (rc || splits == 1) return rc;
  const int64_t n = a.M * a.Ng;
  int64_t blocks = (n + 255) / 256;
  if (blocks > 4096) blocks = 4096;
  hipLaunchKernelGGL(conv_sum_partials, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream,
                     (const float*)workspace, (float*)dw, n, splits);
  return nbk_check_launch("conv_sum_partials");
}
