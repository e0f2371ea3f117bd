// Hand-scheduled kernels for row programs whose generated kernel is bound by the vector ALU and
// not by memory.  Each one computes exactly what its program computes (same operands, same
// results up to the rounding of a differently associated sum) and is attached, by the hash of
// that program, to the entry the generated kernels have in the lookup table; where a launch does
// not meet a kernel's conditions (row length, alignment) the generated forms run as before.
//
// Softmax cross-entropy against integer labels with its gradient, logits and gradient in bf16:
// the program of nabla_amd/ops/xent.py once the planner has merged the forward and the backward
// row program (nabla/nn/functional/losses.py:20-77 in the reference: one-hot, logsoftmax and the
// logsoftmax VJP over tensors the size of the logits).  The generated kernel needs ~57 vector
// instructions per element for it (a library exp twice per element, a column index compared
// with the label at every element); here a row lives in registers as it is stored, exp(x - m)
// is one fused multiply-add and one v_exp_f32, and the label touches one element per row:
// ~10 instructions per element, so the launch is bound by its traffic (1.05 GB in 197 us over
// 8192 x 32000 logits: 5.3 TB/s, the rate of a plain copy of that size).
#include "rowprog_device.h"
#include "rowprog_spec.h"

namespace {

constexpr int XE_BLOCK = 256;   // lanes per row
constexpr int XE_PIECES = 16;   // 16-byte pieces of a row per lane: rows of up to 32768 elements
constexpr float XE_LOG2E = 1.44269504088896340736f;

typedef uint32_t xe_u32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float xe_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float xe_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
typedef float xe_f32x2 __attribute__((ext_vector_type(2)));
typedef __bf16 xe_bf16x2 __attribute__((ext_vector_type(2)));
// two roundings to nearest even in one v_cvt_pk_bf16_f32
__device__ __forceinline__ uint32_t xe_pack(float a, float b) {
  const xe_f32x2 f = {a, b};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f, xe_bf16x2));
}
// max(m, a, b) in one instruction (NaN operands are passed over, as by fmaxf)
__device__ __forceinline__ float xe_max3(float m, float a, float b) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(m), "v"(a), "v"(b));
  return r;
}

// The row stays in registers as stored between the phases: without this the compiler carries the
// unpacked elements (twice the registers) from one phase to the next and spills.
__device__ __forceinline__ void xe_keep_packed(xe_u32x4 (&v)[XE_PIECES]) {
#pragma unroll
  for (int j = 0; j < XE_PIECES; ++j) asm volatile("" : "+v"(v[j]));
}

// operands of the program: 0 logits bf16 [rows, C]; 1 labels int64 per row; 2 loss f32 per row
// (out); 3 scale f32 per row; 4 gradient bf16 [rows, C] (out):
//   m = max_c x;  lse = m + log(sum_c exp(x - m));  loss = lse - x[label]  (0 for a label
//   outside [0, C));  grad = (exp(x - lse) - [c == label]) * scale
template <bool STREAM>
__global__ __launch_bounds__(XE_BLOCK, 4) void rp_hand_xent_bf16_i64(const nbk_rowprog P,
                                                                      int64_t rows) {
  __shared__ float red_buf[64];
  int red_phase = 0;
  const int C = (int)P.C, n16 = C >> 3, lane = threadIdx.x;
  const nbk_operand o0 = P.operand[0], o1 = P.operand[1], o2 = P.operand[2], o3 = P.operand[3],
                    o4 = P.operand[4];
  const int64_t ld1 = P.lead_dim[1], ld2 = P.lead_dim[2], ld3 = P.lead_dim[3];
  struct Row {
    const uint16_t* x;
    int64_t off1, off2, off3, off4;
  };
  auto locate = [&](int64_t row) {
    uint32_t lead_idx[4];
    rp_decompose_row((uint32_t)row, P.n_lead, (uint32_t)ld1, (uint32_t)ld2, (uint32_t)ld3, lead_idx);
    Row r;
    r.x = (const uint16_t*)o0.ptr + rp_row_offset(o0, lead_idx, 4);
    r.off1 = rp_row_offset(o1, lead_idx, 4);
    r.off2 = rp_row_offset(o2, lead_idx, 4);
    r.off3 = rp_row_offset(o3, lead_idx, 4);
    r.off4 = rp_row_offset(o4, lead_idx, 4);
    return r;
  };
  // piece j of a lane sits at (uniform row base + 4096 j) + 16 lane.  The lane offset is made
  // opaque once per row, or the compiler computes the sixteen offsets and bounds of a lane's
  // pieces ahead of the row loop and keeps them in registers (82 registers as it is: five
  // workgroups per CU).
  uint32_t lane_off = (uint32_t)lane * 16u;
  auto request = [&](const Row& r, xe_u32x4& piece, int j) {
    piece = (xe_u32x4)(0xff80ff80u);  // -inf: takes part in nothing
    const xe_u32x4* src = (const xe_u32x4*)((const char*)r.x + (size_t)j * (XE_BLOCK * 16) + lane_off);
    if ((int)(lane_off >> 4) + j * XE_BLOCK < n16) piece = STREAM ? __builtin_nontemporal_load(src) : *src;
  };
  for (int64_t row = blockIdx.x; row < rows; row += gridDim.x) {
    asm volatile("" : "+v"(lane_off));
    const Row cur = locate(row);
    // the whole row is requested at once: up to 64 KB in flight per workgroup, four workgroups
    // to a CU (requesting the next row piece by piece during the gradient phase was measured:
    // the same time, and registers enough to spill)
    xe_u32x4 v[XE_PIECES];
#pragma unroll
    for (int j = 0; j < XE_PIECES; ++j) request(cur, v[j], j);
    const int64_t label = ((const int64_t*)o1.ptr)[cur.off1];
    const bool labelled = (uint64_t)label < (uint64_t)C;
    const float picked = labelled ? nbk_bf16_to_f32(cur.x[label]) : 0.f;
    const float scale = ((const float*)o3.ptr)[cur.off3];

    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < XE_PIECES; ++j)
#pragma unroll
      for (int w = 0; w < 4; ++w) m = xe_max3(m, xe_lo(v[j][w]), xe_hi(v[j][w]));
    xe_keep_packed(v);
    {
      float rv[1] = {m};
      const int rk[1] = {NBK_RED_MAX};
      rp_block_reduce_n(rv, rk, 1, red_buf, red_phase);
      m = rv[0];
    }
    // exp(x - m) = 2^(x log2(e) - m log2(e)): the rounding of m log2(e) scales every term alike
    const float mk = m * XE_LOG2E;
    float s0 = 0.f, s1 = 0.f;
#pragma unroll
    for (int j = 0; j < XE_PIECES; ++j)
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        s0 += __builtin_amdgcn_exp2f(__builtin_fmaf(xe_lo(v[j][w]), XE_LOG2E, -mk));
        s1 += __builtin_amdgcn_exp2f(__builtin_fmaf(xe_hi(v[j][w]), XE_LOG2E, -mk));
      }
    float total = s0 + s1;
    xe_keep_packed(v);
    {
      float rv[1] = {total};
      const int rk[1] = {NBK_RED_SUM};
      rp_block_reduce_n(rv, rk, 1, red_buf, red_phase);
      total = rv[0];
    }
    const float lse = m + logf(total);
    if (lane == 0) ((float*)o2.ptr)[cur.off2] = lse - picked;

    const float lk = lse * XE_LOG2E;
    const int lab16 = labelled ? (int)(label >> 3) : -1, labw = (int)(label & 7);
    char* grad = (char*)((uint16_t*)o4.ptr + cur.off4);
#pragma unroll
    for (int j = 0; j < XE_PIECES; ++j) {
      const int ch = (int)(lane_off >> 4) + j * XE_BLOCK;
      float p[8];
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        p[2 * w] = __builtin_amdgcn_exp2f(__builtin_fmaf(xe_lo(v[j][w]), XE_LOG2E, -lk));
        p[2 * w + 1] = __builtin_amdgcn_exp2f(__builtin_fmaf(xe_hi(v[j][w]), XE_LOG2E, -lk));
      }
      if (ch < n16) {
        if (ch == lab16) {  // one piece of the row holds the label's element
#pragma unroll
          for (int i = 0; i < 8; ++i) p[i] -= (i == labw) ? 1.f : 0.f;
        }
        xe_u32x4 u;
#pragma unroll
        for (int w = 0; w < 4; ++w) u[w] = xe_pack(p[2 * w] * scale, p[2 * w + 1] * scale);
        xe_u32x4* dst = (xe_u32x4*)(grad + (size_t)j * (XE_BLOCK * 16) + lane_off);
        if (STREAM) __builtin_nontemporal_store(u, dst);
        else *dst = u;
      }
    }
  }
}

template __global__ void rp_hand_xent_bf16_i64<false>(const nbk_rowprog, int64_t);
template __global__ void rp_hand_xent_bf16_i64<true>(const nbk_rowprog, int64_t);

}  // namespace

#ifndef __HIP_DEVICE_COMPILE__
// What a launch must meet for the kernel above: rows of whole 16-byte pieces, at most
// XE_PIECES of them per lane and enough of them to occupy the lanes (shorter rows are served
// well by the generated register-resident forms), 16-byte aligned in both row-shaped operands.
static bool xe_fits(const nbk_rowprog* p) {
  if (p->n_operands != 5 || (p->C & 7) != 0 || p->C < 4096 ||
      p->C > (int64_t)XE_BLOCK * XE_PIECES * 8)
    return false;
  for (int i = 0; i < 5; i += 4) {
    const nbk_operand& o = p->operand[i];
    if (o.col_stride != 1 || o.dtype != NBK_BF16 || ((uintptr_t)o.ptr & 15) != 0) return false;
    for (int k = 0; k < p->n_lead; ++k)
      if (o.lead_stride[k] & 7) return false;
  }
  return p->operand[1].dtype == NBK_I64 && p->operand[2].dtype == NBK_F32 &&
         p->operand[3].dtype == NBK_F32;
}

// The program comes in two orders: with the label mask of the gradient phase recomputed (the
// planner does that for masks of 2^22 elements and more) or shared with the loss phase.
extern const rp_hand_entry rp_hand_table[] = {
    {0x32ead8892650fe1bULL, (const void*)rp_hand_xent_bf16_i64<false>,
     (const void*)rp_hand_xent_bf16_i64<true>, XE_BLOCK, xe_fits},
    {0xb23538fd6922ab4fULL, (const void*)rp_hand_xent_bf16_i64<false>,
     (const void*)rp_hand_xent_bf16_i64<true>, XE_BLOCK, xe_fits},
};
extern const int rp_hand_count = (int)(sizeof(rp_hand_table) / sizeof(rp_hand_table[0]));
#endif
