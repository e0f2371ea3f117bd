// Optimizer updates for a whole list of parameters in one launch.
//
// An optimizer step touches every parameter once with the same few lines of arithmetic; issued
// per parameter that is one launch each, most of them far too small to fill the chip (a LoRA
// factor is 32 K elements).  Here the list of tensors travels in the kernel arguments, every
// workgroup finds its tensor and its 16-byte-vector chunk from running block counts, and the
// whole step is one launch that streams param / grad / state in and param / state out once:
// 7 x element size per element for AdamW, 5 x for SGD with momentum, 3 x without.
//
// The arithmetic is that of nabla/nn/optim/functional.py (sgd_step 14-39, adamw_step 116-162):
// fp32 in registers whatever the storage type, one rounding per stored result.
#include "nbk_common.h"

namespace {

constexpr int kBlock = 256;
constexpr int kUnroll = 4;  // 16-byte vectors per lane per chunk

struct MultiArgs {
  int32_t n;
  int32_t first_block[NBK_OPT_MULTI_MAX + 1];
  uint8_t vec_ok[NBK_OPT_MULTI_MAX];  // every pointer of the tensor is 16-byte aligned
  nbk_opt_tensor t[NBK_OPT_MULTI_MAX];
};

struct AdamwParams {
  float lr, beta1, beta2, eps, weight_decay;
  float c1, c2;                // bias corrections when `step` is null
  float log_beta1, log_beta2;  // with `step`: c = 1 - beta^step = -expm1(step * log(beta))
  const float* step;
  int32_t bias_correction;
};

struct SgdParams {
  float lr, momentum, weight_decay;
};

template <typename T>
struct Vec;
template <>
struct Vec<float> {
  static constexpr int N = 4;
  using raw = float4;
  static __device__ __forceinline__ void unpack(const raw& r, float* f) {
    f[0] = r.x; f[1] = r.y; f[2] = r.z; f[3] = r.w;
  }
  static __device__ __forceinline__ raw pack(const float* f) { return make_float4(f[0], f[1], f[2], f[3]); }
  static __device__ __forceinline__ float load1(const float* p) { return *p; }
  static __device__ __forceinline__ void store1(float* p, float v) { *p = v; }
};
template <>
struct Vec<uint16_t> {  // bfloat16
  static constexpr int N = 8;
  using raw = uint4;
  static __device__ __forceinline__ void unpack(const raw& r, float* f) {
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = __uint_as_float(w[i] << 16);
      f[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ raw pack(const float* f) {
    uint32_t w[4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
      w[i] = (uint32_t)nbk_f32_to_bf16(f[2 * i]) | ((uint32_t)nbk_f32_to_bf16(f[2 * i + 1]) << 16);
    return make_uint4(w[0], w[1], w[2], w[3]);
  }
  static __device__ __forceinline__ float load1(const uint16_t* p) { return nbk_bf16_to_f32(*p); }
  static __device__ __forceinline__ void store1(uint16_t* p, float v) { *p = nbk_f32_to_bf16(v); }
};

// One element of AdamW with decoupled decay; (m, v) are updated in place.
struct AdamwRule {
  float lr, b1, b2, one_m_b1, one_m_b2, eps, wd, rc1, rc2;
  static constexpr bool kHasM = true, kHasV = true;
  __device__ __forceinline__ float apply(float p, float g, float& m, float& v) const {
    m = fmaf(m, b1, g * one_m_b1);
    v = fmaf(v, b2, (g * g) * one_m_b2);
    float upd = (m * rc1) / (sqrtf(v * rc2) + eps);
    upd = fmaf(p, wd, upd);
    return fmaf(-upd, lr, p);
  }
};
// SGD: L2 decay joins the gradient; with momentum the buffer (in `m`) becomes
// momentum * buffer + direction and is the direction of the step.
template <bool MOMENTUM>
struct SgdRule {
  float lr, mom, wd;
  static constexpr bool kHasM = MOMENTUM, kHasV = false;
  __device__ __forceinline__ float apply(float p, float g, float& m, float&) const {
    float dir = fmaf(p, wd, g);
    if (MOMENTUM) {
      m = fmaf(mom, m, dir);
      dir = m;
    }
    return fmaf(-dir, lr, p);
  }
};

template <typename T, typename Rule>
__device__ __forceinline__ void update_chunk(const nbk_opt_tensor& t, bool vec_ok, int64_t chunk,
                                             const Rule& rule) {
  using V = Vec<T>;
  constexpr int N = V::N;
  constexpr int64_t kChunk = (int64_t)kBlock * N * kUnroll;
  const T* p = (const T*)t.param;
  const T* g = (const T*)t.grad;
  const T* m = (const T*)t.m;
  const T* v = (const T*)t.v;
  T* po = (T*)t.param_out;
  T* mo = (T*)t.m_out;
  T* vo = (T*)t.v_out;
  const int64_t base = chunk * kChunk;
  const int64_t end = base + kChunk < t.numel ? base + kChunk : t.numel;
  if (vec_ok && end - base == kChunk) {
    typename V::raw rp[kUnroll], rg[kUnroll], rm[kUnroll], rv[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + ((int64_t)u * kBlock + threadIdx.x) * N;
      rp[u] = *(const typename V::raw*)(p + i);
      rg[u] = *(const typename V::raw*)(g + i);
      if (Rule::kHasM) rm[u] = *(const typename V::raw*)(m + i);
      if (Rule::kHasV) rv[u] = *(const typename V::raw*)(v + i);
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int64_t i = base + ((int64_t)u * kBlock + threadIdx.x) * N;
      float fp[N], fg[N], fm[N], fv[N];
      V::unpack(rp[u], fp);
      V::unpack(rg[u], fg);
      if (Rule::kHasM) V::unpack(rm[u], fm);
      if (Rule::kHasV) V::unpack(rv[u], fv);
#pragma unroll
      for (int e = 0; e < N; ++e) {
        float mm = Rule::kHasM ? fm[e] : 0.0f, vv = Rule::kHasV ? fv[e] : 0.0f;
        fp[e] = rule.apply(fp[e], fg[e], mm, vv);
        fm[e] = mm;
        fv[e] = vv;
      }
      *(typename V::raw*)(po + i) = V::pack(fp);
      if (Rule::kHasM) *(typename V::raw*)(mo + i) = V::pack(fm);
      if (Rule::kHasV) *(typename V::raw*)(vo + i) = V::pack(fv);
    }
    return;
  }
  // the last chunk of a tensor, or a tensor at an odd address: element by element
  for (int64_t i = base + threadIdx.x; i < end; i += kBlock) {
    float mm = Rule::kHasM ? V::load1(m + i) : 0.0f, vv = Rule::kHasV ? V::load1(v + i) : 0.0f;
    const float np = rule.apply(V::load1(p + i), V::load1(g + i), mm, vv);
    V::store1(po + i, np);
    if (Rule::kHasM) V::store1(mo + i, mm);
    if (Rule::kHasV) V::store1(vo + i, vv);
  }
}

__device__ __forceinline__ int find_tensor(const MultiArgs& A) {
  int lo = 0, hi = A.n - 1;  // last i with first_block[i] <= blockIdx.x
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if ((int)blockIdx.x >= A.first_block[mid]) lo = mid; else hi = mid - 1;
  }
  return lo;
}

template <typename T>
__global__ __launch_bounds__(kBlock) void adamw_multi_kernel(const MultiArgs A, const AdamwParams P) {
  const int i = find_tensor(A);
  AdamwRule r;
  r.lr = P.lr; r.b1 = P.beta1; r.b2 = P.beta2;
  r.one_m_b1 = 1.0f - P.beta1; r.one_m_b2 = 1.0f - P.beta2;
  r.eps = P.eps; r.wd = P.weight_decay;
  float c1 = P.c1, c2 = P.c2;
  if (P.step != nullptr) {
    const float s = *P.step;
    c1 = -expm1f(s * P.log_beta1);
    c2 = -expm1f(s * P.log_beta2);
  }
  if (!P.bias_correction) c1 = c2 = 1.0f;
  r.rc1 = 1.0f / c1;
  r.rc2 = 1.0f / c2;
  update_chunk<T>(A.t[i], A.vec_ok[i] != 0, (int64_t)blockIdx.x - A.first_block[i], r);
}

template <typename T, bool MOMENTUM>
__global__ __launch_bounds__(kBlock) void sgd_multi_kernel(const MultiArgs A, const SgdParams P) {
  const int i = find_tensor(A);
  SgdRule<MOMENTUM> r;
  r.lr = P.lr; r.mom = P.momentum; r.wd = P.weight_decay;
  update_chunk<T>(A.t[i], A.vec_ok[i] != 0, (int64_t)blockIdx.x - A.first_block[i], r);
}

bool aligned16(const void* p) { return ((uintptr_t)p & 15) == 0; }

// Fills the launch table for tensors [base, base + A.n); returns the block count or -1.
int64_t fill_table(MultiArgs& A, const nbk_opt_tensor* t, int32_t base, int elems_per_vec,
                   bool need_m, bool need_v, const char* who) {
  const int64_t chunk = (int64_t)kBlock * elems_per_vec * kUnroll;
  int64_t blocks = 0;
  for (int i = 0; i < A.n; ++i) {
    const nbk_opt_tensor& x = t[base + i];
    if (!(x.param && x.grad && x.param_out) || (need_m && !(x.m && x.m_out)) ||
        (need_v && !(x.v && x.v_out))) {
      nbk_set_error("%s: tensor %d: null pointer", who, base + i);
      return -1;
    }
    if (x.numel <= 0) {
      nbk_set_error("%s: tensor %d: %lld elements", who, base + i, (long long)x.numel);
      return -1;
    }
    A.vec_ok[i] = aligned16(x.param) && aligned16(x.grad) && aligned16(x.param_out) &&
                  (!need_m || (aligned16(x.m) && aligned16(x.m_out))) &&
                  (!need_v || (aligned16(x.v) && aligned16(x.v_out)));
    A.first_block[i] = (int32_t)blocks;
    blocks += (x.numel + chunk - 1) / chunk;
    if (blocks > 0x7fffffffLL) {
      nbk_set_error("%s: launch too large", who);
      return -1;
    }
    A.t[i] = x;
  }
  A.first_block[A.n] = (int32_t)blocks;
  return blocks;
}

}  // namespace

extern "C" int nbk_adamw_multi(const nbk_adamw_desc* d, const nbk_opt_tensor* tensors, int32_t n,
                               void* stream) {
  NBK_REQUIRE(d != nullptr && tensors != nullptr && n > 0, "adamw_multi: no tensors");
  NBK_REQUIRE(d->dtype == NBK_F32 || d->dtype == NBK_BF16, "adamw_multi: dtype %d", d->dtype);
  NBK_REQUIRE(d->beta1 >= 0.0f && d->beta1 < 1.0f && d->beta2 >= 0.0f && d->beta2 < 1.0f,
              "adamw_multi: betas (%g, %g) outside [0, 1)", d->beta1, d->beta2);
  if (d->bias_correction && d->step == nullptr)
    NBK_REQUIRE(d->c1 > 0.0f && d->c2 > 0.0f, "adamw_multi: bias corrections (%g, %g) must be positive",
                d->c1, d->c2);
  AdamwParams P;
  P.lr = d->lr; P.beta1 = d->beta1; P.beta2 = d->beta2; P.eps = d->eps; P.weight_decay = d->weight_decay;
  P.c1 = d->c1; P.c2 = d->c2; P.log_beta1 = d->log_beta1; P.log_beta2 = d->log_beta2;
  P.step = d->step; P.bias_correction = d->bias_correction;
  for (int32_t base = 0; base < n; base += NBK_OPT_MULTI_MAX) {
    MultiArgs A;
    A.n = n - base < NBK_OPT_MULTI_MAX ? n - base : NBK_OPT_MULTI_MAX;
    const int64_t blocks = fill_table(A, tensors, base, d->dtype == NBK_F32 ? 4 : 8, true, true, "adamw_multi");
    if (blocks < 0) return NBK_ERR_INVALID;
    if (d->dtype == NBK_F32)
      hipLaunchKernelGGL(adamw_multi_kernel<float>, dim3((unsigned)blocks), dim3(kBlock), 0,
                         (hipStream_t)stream, A, P);
    else
      hipLaunchKernelGGL(adamw_multi_kernel<uint16_t>, dim3((unsigned)blocks), dim3(kBlock), 0,
                         (hipStream_t)stream, A, P);
  }
  return nbk_check_launch("adamw_multi_kernel");
}

extern "C" int nbk_sgd_multi(const nbk_sgd_desc* d, const nbk_opt_tensor* tensors, int32_t n,
                             void* stream) {
  NBK_REQUIRE(d != nullptr && tensors != nullptr && n > 0, "sgd_multi: no tensors");
  NBK_REQUIRE(d->dtype == NBK_F32 || d->dtype == NBK_BF16, "sgd_multi: dtype %d", d->dtype);
  const bool mom = d->momentum != 0.0f;
  SgdParams P;
  P.lr = d->lr; P.momentum = d->momentum; P.weight_decay = d->weight_decay;
  for (int32_t base = 0; base < n; base += NBK_OPT_MULTI_MAX) {
    MultiArgs A;
    A.n = n - base < NBK_OPT_MULTI_MAX ? n - base : NBK_OPT_MULTI_MAX;
    const int64_t blocks = fill_table(A, tensors, base, d->dtype == NBK_F32 ? 4 : 8, mom, false, "sgd_multi");
    if (blocks < 0) return NBK_ERR_INVALID;
    const dim3 grid((unsigned)blocks), block(kBlock);
    hipStream_t s = (hipStream_t)stream;
    if (d->dtype == NBK_F32) {
      if (mom) hipLaunchKernelGGL((sgd_multi_kernel<float, true>), grid, block, 0, s, A, P);
      else hipLaunchKernelGGL((sgd_multi_kernel<float, false>), grid, block, 0, s, A, P);
    } else {
      if (mom) hipLaunchKernelGGL((sgd_multi_kernel<uint16_t, true>), grid, block, 0, s, A, P);
      else hipLaunchKernelGGL((sgd_multi_kernel<uint16_t, false>), grid, block, 0, s, A, P);
    }
  }
  return nbk_check_launch("sgd_multi_kernel");
}
