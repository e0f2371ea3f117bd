/*
 * nbk.h -- C ABI of libnbk.so, the gfx950 kernel library behind the nabla_amd
 * execution backend.
 *
 * The reference (nabla-ml/nabla) has no native code of its own: every
 * Operation.kernel() calls a `max.graph.ops.*` builder and the engine hands the
 * finished graph to `InferenceSession.load(graph)` / `model(*buffers)`
 * (nabla/core/graph/engine.py:656-663).  This header is what replaces those
 * MAX call sites on one MI355X.  Each entry point cites the reference call site
 * whose arithmetic it takes over.
 *
 * Conventions
 *   - plain pointers and sizes only; device pointers are raw HIP addresses
 *   - every launch goes onto the hipStream_t passed as `void* stream`
 *     (NULL = the legacy default stream)
 *   - kernels never allocate: the caller owns inputs, outputs and workspace
 *   - return value: 0 on success, negative nbk_status otherwise;
 *     nbk_last_error() returns a thread-local message for the last failure
 *   - mutable global state is limited to that message (thread-local) and to
 *     mutex-guarded caches that are filled on first use: the table of
 *     specialised row kernels, per-kernel occupancy, loaded user libraries
 */
#ifndef NBK_H_
#define NBK_H_

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* ------------------------------------------------------------------ status */
enum nbk_status {
  NBK_OK = 0,
  NBK_ERR_INVALID = -1,   /* bad argument (shape, dtype, alignment, limits) */
  NBK_ERR_LAUNCH = -2,    /* HIP reported a launch / runtime error          */
  NBK_ERR_UNSUPPORTED = -3
};

/* ------------------------------------------------------------------ dtypes */
enum nbk_dtype {
  NBK_F32 = 0,
  NBK_BF16 = 1,
  NBK_F16 = 2,
  NBK_I32 = 3,
  NBK_I64 = 4,
  NBK_U8 = 5    /* also bool: 0 / 1 */
};

/* --------------------------------------------------------------- lifecycle */
/* Select the device, query it, and make sure it is a gfx950 part.
 * Replaces the session singleton of nabla/core/common/context.py:120-139. */
int nbk_init(int device);
const char* nbk_last_error(void);
/* ABI version of this header; the ctypes shim refuses a mismatch. */
int nbk_abi_version(void);
#define NBK_ABI_VERSION 24

/* ===================================================================== */
/*  Row programs: fused elementwise chains + last-axis reductions         */
/* ===================================================================== */
/*
 * One kernel family executes every fused group of elementwise ops
 * (nabla/ops/binary.py:18-156, unary.py:20-697, comparison.py:63-130,
 * control_flow.py:21-141 WhereOp, creation.py fills/arange/tril) together
 * with the single-axis keepdims reductions over the LAST axis that the
 * reference emits as ops.sum / ops.mean / ops._reduce_max
 * (nabla/ops/reduction.py:147-245), including softmax / logsoftmax
 * (unary.py:192-230, 598-632) and layer_norm (nn/functional/layers.py:38-56)
 * once the lowering pass has fused their primitive ops.
 *
 * Iteration domain: rows x C, rows = prod(lead_dim[0..n_lead)).
 * An operand is addressed as
 *     ptr[ sum_k lead_idx[k]*lead_stride[k] + col*col_stride ]   (elements)
 * so broadcasts (stride 0), row vectors (col_stride 0), column vectors
 * (all lead strides 0) and transposed views are all the same thing.
 *
 * The program is a stream of 8-byte instructions interpreted by every lane.
 * Registers: 16 vector registers (4 consecutive columns each) numbered 0..15
 * and 16 per-row scalar registers numbered 16..31.  A program is
 *     { prologue ; BODY n ; n body instructions } ... HALT
 * Prologue instructions run once per row on scalar registers; body
 * instructions run once per 4-column chunk.
 */
#define NBK_RP_MAX_OPERANDS 20
#define NBK_RP_MAX_INS 224
#define NBK_RP_MAX_IMM 24
#define NBK_RP_MAX_LEAD 4
#define NBK_RP_NVEC 16
#define NBK_RP_NSCL 16
#define NBK_RP_NACC 4
#define NBK_RP_MAX_STAGE 4

typedef struct nbk_operand {
  void* ptr;                           /* device address of element 0          */
  int64_t lead_stride[NBK_RP_MAX_LEAD];/* element strides of the leading dims  */
  int32_t col_stride;                  /* element stride along the row axis    */
  int32_t dtype;                       /* nbk_dtype                            */
  int32_t vec_ok;                      /* 1: 4 columns can move as one access  */
  int32_t stage_slot;                  /* >=0: row is pre-loaded into LDS slot */
} nbk_operand;

typedef struct nbk_ins {
  uint8_t op;    /* nbk_rp_op                                         */
  uint8_t dst;   /* register, accumulator index or operand index      */
  uint8_t a, b, c; /* source registers / operand index / immediate id */
  uint8_t pad;
  uint16_t aux;  /* BODY: number of body instructions                 */
} nbk_ins;

enum nbk_rp_op {
  NBK_OP_HALT = 0,
  /* structure */
  NBK_OP_BODY = 1,     /* aux = body length                                    */
  /* memory (a = operand index) */
  NBK_OP_LDG = 2,      /* body: vreg dst <- operand a, 4 columns               */
  NBK_OP_STG = 3,      /* body: operand dst <- vreg a                          */
  NBK_OP_LDR = 4,      /* prologue: sreg dst <- operand a at column 0          */
  NBK_OP_STR = 5,      /* prologue: operand dst <- sreg a (column 0, 1 lane)   */
  NBK_OP_IMM = 6,      /* prologue: sreg dst <- imm[a]                         */
  NBK_OP_COLIDX = 7,   /* body: vreg dst <- column index, as float (a = 0) or int32 (a = 1) */
  NBK_OP_LEADIDX = 8,  /* prologue: sreg dst <- index along leading dim a, as float (b = 0) or int32 (b = 1) */
  /* reductions over the row */
  NBK_OP_ACCINIT = 9,  /* prologue: acc dst <- identity of kind a              */
  NBK_OP_ACC = 10,     /* body: acc dst <- combine(acc, vreg a), kind b        */
  NBK_OP_RED = 11,     /* prologue: sreg dst <- block-reduce(acc a), kind b    */
  /* unary  dst <- f(a) */
  NBK_OP_MOV = 16, NBK_OP_NEG = 17, NBK_OP_RELU = 18, NBK_OP_EXP = 19,
  NBK_OP_LOG = 20, NBK_OP_SQRT = 21, NBK_OP_RSQRT = 22, NBK_OP_ERF = 23,
  NBK_OP_GELU = 24, NBK_OP_TANH = 25, NBK_OP_SIGMOID = 26, NBK_OP_ABS = 27,
  NBK_OP_RBF16 = 28,   /* round to bf16 and back                               */
  NBK_OP_NOT = 29,     /* 1 - a  on 0/1 values                                 */
  NBK_OP_TRUNC = 30,   /* round toward zero (float -> integer casts)           */
  NBK_OP_NEZ = 31,     /* a != 0 -> 1/0 (casts to bool)                        */
  /* binary dst <- f(a, b) */
  NBK_OP_ADD = 32, NBK_OP_SUB = 33, NBK_OP_MUL = 34, NBK_OP_DIV = 35,
  NBK_OP_MAX = 36, NBK_OP_MIN = 37, NBK_OP_GT = 38, NBK_OP_GE = 39,
  NBK_OP_EQ = 40, NBK_OP_NE = 41, NBK_OP_LT = 42, NBK_OP_LE = 43,
  NBK_OP_POW = 44, NBK_OP_AND = 45, NBK_OP_OR = 46,
  /* ternary */
  NBK_OP_WHERE = 48,   /* dst <- a != 0 ? b : c                                */
  NBK_OP_FMA = 49,     /* dst <- a * b + c                                     */
  /* more unary ops (the block 16..31 is full) */
  NBK_OP_DGELU = 50,   /* derivative of the exact GELU: Phi(a) + a * phi(a)    */
  NBK_OP_SIN = 51, NBK_OP_COS = 52, /* unary; the block 16..31 is full             */
  /* Integer registers.  A register is 32 bits; the program decides what they mean.  Values of
   * integer tensors are loaded, held and stored as two's-complement int32 (LDG / LDR / STG /
   * STR go by the operand's dtype), and these instructions compute on them exactly, wrapping
   * modulo 2^32.  An int64 operand is read SATURATED to the int32 range and written sign-
   * extended: exact for comparisons with an index or constant strictly inside that range,
   * which is the one use of int64 tensors the lowering leaves in row programs; arithmetic on
   * int64 values belongs to nbk_ew_int64.  Floats, bool and uint8 are fp32 in registers.  MOV,
   * WHERE (its payload) and IMM move bits and serve both; an integer immediate is stored in
   * imm[] by its bit pattern. */
  /* binary on int32 (comparisons produce a float 0 / 1, like their float forms) */
  NBK_OP_IADD = 64, NBK_OP_ISUB = 65, NBK_OP_IMUL = 66, NBK_OP_IMAX = 67, NBK_OP_IMIN = 68,
  NBK_OP_IGT = 69, NBK_OP_IGE = 70, NBK_OP_IEQ = 71, NBK_OP_INE = 72, NBK_OP_ILT = 73,
  NBK_OP_ILE = 74,
  /* unary on int32 */
  NBK_OP_INEG = 80, NBK_OP_IABS = 81, NBK_OP_IRELU = 82,
  NBK_OP_I2F = 83,     /* int32 -> float                                        */
  NBK_OP_F2I = 84,     /* float -> int32, toward zero                           */
  NBK_OP_INEZ = 85     /* int32 != 0 -> float 1 / 0                             */
};

enum nbk_red_kind { NBK_RED_SUM = 0, NBK_RED_MAX = 1, NBK_RED_MIN = 2 };

typedef struct nbk_rowprog {
  int64_t lead_dim[NBK_RP_MAX_LEAD];
  int64_t C;              /* row length                                        */
  int32_t n_lead;
  int32_t n_operands;
  int32_t n_ins;
  int32_t n_imm;
  int32_t has_reduce;     /* 0: flat launch, 1: one workgroup per row          */
  int32_t block;          /* workgroup size for has_reduce=1 (64..512, pow2)   */
  int32_t n_stage;        /* operands pre-loaded into LDS (has_reduce=1 only)  */
  int32_t reserved;       /* 1: run on the interpreter even if a specialised kernel exists */
  float imm[NBK_RP_MAX_IMM];
  nbk_operand operand[NBK_RP_MAX_OPERANDS];
  nbk_ins ins[NBK_RP_MAX_INS];
} nbk_rowprog;

int nbk_rowprog_launch(const nbk_rowprog* prog, void* stream);
/* 1 if the library carries a straight-line (ahead-of-time specialised) kernel
 * for this program, 2 if it also carries a hand-scheduled kernel that this launch
 * (row length, alignment) would take, 0 if the interpreter will run it.  Results
 * are the same to rounding either way; NBK_ROWPROG_INTERPRET=1 forces the
 * interpreter, NBK_ROWPROG_HAND=0 the generated kernels. */
int nbk_rowprog_is_specialized(const nbk_rowprog* prog);
/* The 64-bit hash (FNV-1a over header, operand classes, instructions, immediates; pointers,
 * strides and extents excluded) by which a program finds its specialised kernel.  That
 * kernel's name ends in the hash in hex, so a profile can be matched to the program it is
 * for.  0 for an invalid program. */
uint64_t nbk_rowprog_hash(const nbk_rowprog* prog);

/* ===================================================================== */
/*  Reductions over a middle / leading axis                               */
/* ===================================================================== */
/* in: contiguous [outer, red, inner] -> out: contiguous [outer, inner].
 * Covers the inner>1 cases of nabla/ops/reduction.py:147-245 that the
 * autodiff un-broadcast emits (nabla/core/autograd/backward.py:31-54),
 * e.g. bias and layer-norm weight gradients.  kind: nbk_red_kind. */
int nbk_reduce_mid(const void* in, void* out, int32_t dtype_in, int32_t dtype_out,
                   int64_t outer, int64_t red, int64_t inner, int32_t kind,
                   void* stream);
/* Several independent reductions of that form in one launch (the un-broadcast sums of a
 * backward pass -- one per bias and norm parameter -- are many, small and ready together).
 * `tasks` is a host array; results are those of nbk_reduce_mid task by task. */
#define NBK_REDUCE_BATCH_MAX 24   /* tasks per launch; longer lists take several */
typedef struct nbk_reduce_task {
  const void* in;
  void* out;
  int64_t outer, red, inner;
  int32_t dtype_in, dtype_out, kind, reserved;
} nbk_reduce_task;
int nbk_reduce_mid_batch(const nbk_reduce_task* tasks, int32_t n, void* stream);

/* ===================================================================== */
/*  Strided copy (materialise a view)                                     */
/* ===================================================================== */
/* dst (contiguous, row-major over shape) <- src viewed with src_stride.
 * Serves permute / swap_axes / broadcast_to / slice_tensor / pad /
 * concatenate / slice_update when a consumer cannot fold the view
 * (nabla/ops/view/shape.py:56-158, 586-980, 1313-1398; view/axes.py:43-868).
 * dst_stride may also be strided (writes into a window of a larger buffer). */
#define NBK_MAX_RANK 8
int nbk_copy_strided(const void* src, void* dst, int32_t dtype_src, int32_t dtype_dst,
                     int32_t rank, const int64_t* shape, const int64_t* src_stride,
                     const int64_t* dst_stride, void* stream);
/* Fill a contiguous buffer with a constant (creation.py:50-93). */
int nbk_fill(void* dst, int32_t dtype, int64_t n, double value, void* stream);

/* ===================================================================== */
/*  GEMM                                                                  */
/* ===================================================================== */
/* C[b] = act(alpha * op(A[b]) @ op(B[b]) + bias) (+ or x) residual; replaces ops.matmul at nabla/ops/binary.py:198 for the forward
 * product and for both backward products of MatmulOp.vjp_rule
 * (binary.py:303-314), whose swap_axes are folded into the strides here.
 * A is M x K with element strides (a_rs, a_cs), B is K x N with (b_rs, b_cs);
 * one of the two strides of each must be 1.  C is row-major with leading
 * dimension ldc.  Batches are strided (stride 0 = broadcast).
 * `batch_reduce` != 0 sums the products of all batches into ONE C
 * (dW of a 3-D activation against a 2-D weight: backward.py:36-41).
 * dtype_ab: NBK_F32 or NBK_BF16; accumulation is always fp32. */
enum nbk_gemm_act { NBK_ACT_NONE = 0, NBK_ACT_RELU = 1, NBK_ACT_GELU = 2 };
/* what the residual does to the result: added (x + r: a skip connection, an accumulated
 * gradient) or multiplied in (x * r: the saved derivative of an activation, a mask) */
enum nbk_gemm_residual_op { NBK_RES_ADD = 0, NBK_RES_MUL = 1 };
/* second result of the same launch: C_aux = act'(alpha * op(A) @ op(B) + bias), the derivative of
 * the activation at the value the activation was applied to (what the backward pass of
 * gelu(x @ W + b) multiplies the cotangent with: nabla/ops/unary.py:567-595), taken from the
 * fp32 accumulator like C itself, so that the pre-activation never makes a trip through memory */
enum nbk_gemm_aux_op { NBK_AUX_NONE = 0, NBK_AUX_ACT_GRAD = 1 };
#define NBK_GEMM_MAX_TERMS 4
typedef struct nbk_gemm_term {
  const void* A; const void* B;
  int64_t K, a_rs, a_cs, b_rs, b_cs;
} nbk_gemm_term;
typedef struct nbk_gemm_desc {
  const void* A; const void* B; void* C;
  const void* bias;      /* NULL or [N] (dtype_c), added to every row        */
  const void* residual;  /* NULL or same layout as C, applied after activation */
  int64_t M, N, K;
  int64_t a_rs, a_cs, b_rs, b_cs, ldc;
  int64_t batch, a_bs, b_bs, c_bs;
  /* Second batch level: batch index z = zo * batch_inner + zi; operand offsets are
   * zo * x_bs + zi * x_bs2 (batch_inner <= 1: one level, the *_bs2 are ignored).
   * This is how [B, S, H, hd] heads are read and written as [B, H] batches of
   * S x hd matrices without a transposing copy. */
  int64_t batch_inner, a_bs2, b_bs2, c_bs2;
  int32_t dtype_ab, dtype_c;
  int32_t act;
  int32_t batch_reduce;
  float alpha;
  int32_t residual_op;   /* enum nbk_gemm_residual_op */
  void* C_aux;           /* NULL or a second result in C's layout and dtype (see nbk_gemm_aux_op) */
  int32_t aux_op;        /* enum nbk_gemm_aux_op; needs act != NBK_ACT_NONE and no residual */
  int32_t reserved;
  /* NULL, or [batch][N] in dtype_c: sum over k of B[b][k][n], a third result of the same launch.
   * With A = x^T and B = dy the product is the weight gradient of a linear layer and this is its
   * bias gradient (the reduction of the cotangent to the bias' shape,
   * nabla/core/autograd/backward.py:31-54), taken from the B fragments the product has in
   * registers, so dy is read once.  bf16 operands, both row-contiguous (a_rs == b_cs == 1) and
   * 16-byte aligned, K % 64 == 0, M % 8 == 0, N % 8 == 0, alpha 1, no bias / residual / activation;
   * anything else is an error.  Row b of the sums belongs to batch index b of the launch, also with
   * two batch levels (b = outer * batch_inner + inner). */
  void* colsum;
  /* n_terms > 0: more operand pairs whose products join the accumulator before the epilogue,
   *   C = act(alpha * (A @ B + sum_i term[i].A @ term[i].B) + bias) ...
   * term[i].A is M x term[i].K with strides (a_rs, a_cs), term[i].B is term[i].K x N with
   * (b_rs, b_cs), one unit stride each.  Two uses: the update of a low-rank adapter inside its
   * base product, x @ W + (x @ A) @ B (nabla/nn/finetune/lora.py:55-79), and a gradient that
   * several products contribute to, dq @ Wq^T + dk @ Wk^T + dv @ Wv^T (the cotangent
   * accumulation of nabla/core/autograd/backward.py:31-54 over MatmulOp.vjp_rule,
   * nabla/ops/binary.py:303-314): the sum is rounded once and no partial result makes a trip
   * through memory.  bf16 operands, batch 1, no column sums.  Inside one launch when every pair
   * is laid out like A and B (same unit-stride side) and 16-byte aligned, with at most two
   * shallow pairs (K <= 64, K % 8 == 0: one K tile each) and at most two deep ones (K % 64 == 0
   * and exactly the strides of A and B: their tiles follow those of A and B); otherwise one
   * launch per pair, each adding itself to the result of the one before (plain products only:
   * no bias, residual, activation or alpha then). */
  int32_t n_terms;
  int32_t reserved2;
  nbk_gemm_term term[NBK_GEMM_MAX_TERMS];
} nbk_gemm_desc;
int nbk_gemm(const nbk_gemm_desc* d, void* stream);

/* C = alpha * A @ W or alpha * A @ W^T for a weight W [w_rows, w_cols] that is stored NF4-coded
 * as quantize_nf4 leaves it (nabla/nn/finetune/qlora.py:41-75): `codes`, one uint8 per weight in
 * row-major order holding the index of one of the sixteen levels (18-38), and `scales`, one fp32
 * per `block` consecutive codes.  Replaces dequantize_nf4 followed by matmul (77-113) and the
 * input-gradient product of that matmul: the dense weight is never built, the kernel reads
 * the codes, looks the levels up, applies the block scale and feeds the matrix cores (bf16: the
 * product level * scale is rounded to bf16 once).  A is row-major [M, K] with leading dimension
 * lda, C row-major [M, N]; dtype (NBK_BF16 or NBK_F32) is the type of A and C.  w_cols and block
 * must be multiples of 8, codes 8-byte aligned. */
typedef struct nbk_gemm_nf4_desc {
  const void* A; const void* codes; const void* scales; void* C;
  int64_t M, w_rows, w_cols;
  int64_t lda, ldc;
  int32_t block;
  int32_t transpose_w;   /* 0: C = A @ W (K = w_rows), 1: C = A @ W^T (K = w_cols) */
  int32_t dtype;
  float alpha;
} nbk_gemm_nf4_desc;
int nbk_gemm_nf4(const nbk_gemm_nf4_desc* d, void* stream);

/* ===================================================================== */
/*  Convolution / pooling (NHWC x HWIO)                                   */
/* ===================================================================== */
/* Replaces ops.conv2d at nabla/ops/convolution.py:252 and the two products
 * of Conv2DOp.vjp_rule (convolution.py:309-392): dgrad (the conv2d_transpose
 * + pad + slice sequence) and wgrad (the conv of permuted tensors).
 * x [N,H,W,Cin], w [R,S,Cin,Cout], y [N,Ho,Wo,Cout]; fp32; dilation 1,
 * groups 1 as the reference validates (convolution.py:602-696). */
typedef struct nbk_conv_desc {
  int64_t N, H, W, Cin, R, S, Cout, Ho, Wo;
  int32_t stride_h, stride_w;
  int32_t pad_t, pad_b, pad_l, pad_r;
  int32_t dtype;      /* NBK_F32 */
  /* forward only: NBK_ACT_NONE, or NBK_ACT_RELU for y = max(conv(x, w) + bias, 0) -- the relu that
   * follows a convolution layer (nabla/ops/unary.py:31-42), applied to the accumulator on its way
   * out; its mask in the backward pass, (pre-activation > 0), equals (y > 0).  The two gradient
   * entry points want NBK_ACT_NONE. */
  int32_t act;
} nbk_conv_desc;
int nbk_conv2d_fwd(const nbk_conv_desc* d, const void* x, const void* w,
                   const void* bias, void* y, void* stream);
int nbk_conv2d_dgrad(const nbk_conv_desc* d, const void* dy, const void* w,
                     void* dx, void* stream);
/* The filter gradient contracts over every output pixel of the batch, so it is
 * computed in K slices whose partial sums go to `workspace` (device memory,
 * 16-byte aligned, nbk_conv2d_wgrad_workspace(d) bytes; contents undefined on
 * return) and are then added in a fixed order.  With workspace == NULL or too
 * small the product runs unsplit: same result up to summation order, slower. */
int64_t nbk_conv2d_wgrad_workspace(const nbk_conv_desc* d);
int nbk_conv2d_wgrad(const nbk_conv_desc* d, const void* x, const void* dy,
                     void* dw, void* workspace, int64_t workspace_bytes, void* stream);

/* max_pool2d forward/backward; replaces the per-window slice + reduce_max +
 * stack graph of nabla/ops/pooling.py:53-137.  Backward follows the
 * reduce_max tie rule (reduction.py:219-230): every element equal to the
 * window maximum receives the full cotangent.  Windows are clipped at the
 * padded border (pooling.py:111-130). */
typedef struct nbk_pool_desc {
  int64_t N, H, W, C, Ho, Wo;
  int32_t kh, kw, stride_h, stride_w, pad_t, pad_l;
  int32_t dtype;
  int32_t reserved;
} nbk_pool_desc;
int nbk_maxpool2d_fwd(const nbk_pool_desc* d, const void* x, void* y, void* stream);
int nbk_maxpool2d_bwd(const nbk_pool_desc* d, const void* x, const void* y,
                      const void* dy, void* dx, void* stream);
/* avg_pool2d forward/backward (nabla/ops/pooling.py:77-110, 140-173): the input is
 * zero-padded first and every window sum is divided by kh * kw, padding included. */
int nbk_avgpool2d_fwd(const nbk_pool_desc* d, const void* x, void* y, void* stream);
int nbk_avgpool2d_bwd(const nbk_pool_desc* d, const void* dy, void* dx, void* stream);

/* ===================================================================== */
/*  Fused attention                                                       */
/* ===================================================================== */
/* O = softmax(mask(Q K^T * scale)) V in one kernel, and its gradients in three;
 * replaces the matmul / mul / where / softmax / matmul graph that
 * scaled_dot_product_attention builds (nabla/nn/functional/layers.py:106-153) and
 * the VJP graphs of those ops, for the case without an explicit mask or dropout.
 * The S x S scores and probabilities are never stored: the forward keeps one
 * log-sum-exp per score row (lse, fp32 [B, H, S]) and the backward recomputes.
 * Tensors are [B, S, H, hd] addressed through element strides (sb, ss, sh) with
 * hd contiguous, so heads are read and written in place of a transpose.
 * dtype NBK_BF16, hd 64 or 128, S a multiple of 128; pointers 16-byte aligned,
 * strides multiples of 8.  causal != 0 masks key > query. */
typedef struct nbk_attn_desc {
  int64_t B, H, S, hd;
  float scale;
  int32_t causal;
  int32_t dtype;
  int32_t reserved;
} nbk_attn_desc;
typedef struct nbk_attn_tensor {
  void* ptr;
  int64_t sb, ss, sh;
} nbk_attn_tensor;
/* `o_lo` (may be NULL, or have ptr == NULL): a second bf16 tensor of O's shape that receives
 * what rounding O to bf16 cut off, O_fp32 - O_bf16.  The backward pass forms
 * delta = rowsum(dO * O) and then dS = P * (dP - delta); where the keys a query sees have
 * values with a large common part, dP - delta cancels most of dP and a delta taken from bf16 O
 * alone puts errors of several percent on dQ and dK (measured: 2-4 % on the query-side
 * gradients of a 12-layer decoder against 0.5-1 % on the value side).  Handing the same tensor
 * to the backward pass brings delta to about 16 bits. */
int nbk_attention_fwd(const nbk_attn_desc* d, const nbk_attn_tensor* q,
                      const nbk_attn_tensor* k, const nbk_attn_tensor* v,
                      const nbk_attn_tensor* o, const nbk_attn_tensor* o_lo, void* lse,
                      void* stream);
/* Backward needs nbk_attention_bwd_workspace(d) bytes of caller scratch (one
 * fp32 per score row: rowsum(dO * O)). */
int64_t nbk_attention_bwd_workspace(const nbk_attn_desc* d);
int nbk_attention_bwd(const nbk_attn_desc* d, const nbk_attn_tensor* q,
                      const nbk_attn_tensor* k, const nbk_attn_tensor* v,
                      const nbk_attn_tensor* o, const nbk_attn_tensor* o_lo, const void* lse,
                      const nbk_attn_tensor* dout, const nbk_attn_tensor* dq,
                      const nbk_attn_tensor* dk, const nbk_attn_tensor* dv,
                      void* workspace, int64_t workspace_bytes, void* stream);

/* The same backward pass for callers that cannot allocate device memory or hand over a
 * workspace: code under HIP graph capture, tight serving loops, harnesses that forbid
 * hipMalloc.  It has no counterpart in the reference.  The row sums live in scratch that is
 * part of the library image (NBK_ATTN_STATIC_ROWS floats = 4 MiB per GPU, held until the
 * process ends); the call allocates nothing and fails with NBK_ERR_INVALID when
 * B * H * S > NBK_ATTN_STATIC_ROWS.  Results are those of nbk_attention_bwd bit for bit.
 * All calls on one GPU share that scratch: calls that overlap in time on one GPU (two streams)
 * race; calls on one stream, or ordered by events, do not.  Nothing needs clearing between
 * calls (each call writes every row it later reads). */
#define NBK_ATTN_STATIC_ROWS (1 << 20)
int nbk_attention_bwd_static(const nbk_attn_desc* d, const nbk_attn_tensor* q,
                             const nbk_attn_tensor* k, const nbk_attn_tensor* v,
                             const nbk_attn_tensor* o, const nbk_attn_tensor* o_lo,
                             const void* lse,
                             const nbk_attn_tensor* dout, const nbk_attn_tensor* dq,
                             const nbk_attn_tensor* dk, const nbk_attn_tensor* dv,
                             void* stream);

/* ===================================================================== */
/*  Index ops (bit-exact)                                                 */
/* ===================================================================== */
/* out[o, j, i] = table[o, idx[j], i]; replaces ops.gather at
 * nabla/ops/view/indexing.py:171 (embedding: nn/functional/layers.py:84-98).
 * Negative indices wrap once; out-of-range indices are an error reported
 * through `status` (a device int32 the caller zeroes; set to 1 on error). */
int nbk_gather(const void* table, const void* idx, void* out, int32_t dtype,
               int32_t idx_dtype, int64_t outer, int64_t axis_len, int64_t n_idx,
               int64_t inner, int32_t* status, void* stream);
/* out[o, idx[j], i] = upd[o, j, i] on top of what `out` already holds (the caller copies x
 * there first); replaces ops.scatter at nabla/ops/view/indexing.py:185-447, which the VJP of
 * gather uses (173-182).  A row named more than once takes the update at the largest j
 * (numpy's assignment rule; the reference leaves that order to its backend).  `winner` is
 * axis_len int32 of caller scratch.  Index wrapping and range errors as in nbk_gather. */
int nbk_scatter(const void* idx, const void* upd, void* out, int32_t dtype, int32_t idx_dtype,
                int64_t outer, int64_t axis_len, int64_t n_idx, int64_t inner,
                int32_t* winner, int32_t* status, void* stream);
/* out[r] = index of the first maximum of in[r, 0..C) as int64; replaces
 * ops.argmax at nabla/ops/reduction.py:745-765. */
int nbk_argmax_rows(const void* in, int64_t* out, int32_t dtype, int64_t rows,
                    int64_t C, int32_t want_min, void* stream);

/* ===================================================================== */
/*  Custom kernels                                                        */
/* ===================================================================== */
/* Contract of a user kernel library loaded by call_custom_kernel
 * (nabla/ops/utils.py:765-824; tests/mojo/kernels/custom_kernel.mojo:12-26):
 * a shared object exporting, per registered name,
 *     int <name>(const nbk_tensor* in, int n_in,
 *                nbk_tensor* out, int n_out, void* stream);
 * nbk_custom() resolves and calls it, and verifies the symbol exists. */
typedef struct nbk_tensor {
  void* ptr;
  int32_t dtype;
  int32_t rank;
  int64_t shape[NBK_MAX_RANK];
  int64_t stride[NBK_MAX_RANK];
} nbk_tensor;
typedef int (*nbk_custom_fn)(const nbk_tensor* in, int n_in, nbk_tensor* out,
                             int n_out, void* stream);
int nbk_custom(const char* library_path, const char* name, const nbk_tensor* in,
               int n_in, nbk_tensor* out, int n_out, void* stream);

/* ===================================================================== */
/*  Elementwise arithmetic on 64-bit integers                             */
/* ===================================================================== */
/* out = op(in[0] [, in[1] [, in[2]]]) element by element in int64 arithmetic; replaces the MAX
 * elementwise ops behind nabla/ops/binary.py:18-156 (add/sub/mul/div), comparison.py:63-106,
 * control_flow.py:21-141 (where) and the casts of unary.py:660-697 whenever an operand or the
 * result is int64 (argmax results, token ids, labels, counters).  The fused row programs hold
 * integers in 32-bit registers, so the lowering sends these operations here instead: exact
 * over the whole int64 range, sums / differences / products wrap modulo 2^64 as numpy's do,
 * division rounds toward zero (x / 0 gives 0).  `op` is one of the NBK_OP_* elementwise codes
 * MOV TRUNC NEG ABS RELU NOT NEZ ADD..OR WHERE FMA.  Every operand has the result's rank and
 * shape (broadcast axes have stride 0; strides in elements) and any dtype: integers and bool
 * widen to int64, floats are cut toward zero.  An operand with ptr == NULL is the constant
 * imm[k].  The result is stored as out->dtype: int64, int32 (low 32 bits), bool (!= 0) or a
 * float type (nearest). */
int nbk_ew_int64(int32_t op, const nbk_tensor* in, const int64_t* imm, int32_t n_in,
                 const nbk_tensor* out, void* stream);

/* ===================================================================== */
/*  Random tensors                                                        */
/* ===================================================================== */
/* The reference's uniform / gaussian (nabla/ops/creation.py:152-183, 462-520) and the dropout
 * mask built on them (nabla/nn/functional/layers.py:64-76: uniform(shape) > p) draw from MAX's
 * generator and thread a seed value through every compiled graph (core/graph/engine.py:80,
 * 610-611).  Here the generator is Philox4x32-10 and the state is two int64 in device memory
 * owned by the caller: state[0] the seed, state[1] the number of steps drawn so far.  Element i
 * of a tensor is word i % 4 of the block with counter (i / 4 low, i / 4 high, stream_id,
 * state[1] low) and key (seed low, seed high): `stream_id` tells the random tensors of one step
 * apart, nbk_rng_advance (state[1] += 1, as a kernel, so that it can be part of a recorded
 * sequence) goes once at the end of a step that drew numbers.
 *   NBK_RANDOM_UNIFORM: a + (b - a) u,  u = (word >> 8) 2^-24 in [0, 1)
 *   NBK_RANDOM_NORMAL:  a + b z, Box-Muller on the word pairs (0, 1) and (2, 3) of a block
 *   NBK_RANDOM_KEEP:    u > a as 1 / 0 (the keep mask of dropout with rate a); also into bool
 * dtype: NBK_F32, NBK_BF16, NBK_F16 (NBK_U8 for KEEP). */
enum nbk_random_mode { NBK_RANDOM_UNIFORM = 0, NBK_RANDOM_NORMAL = 1, NBK_RANDOM_KEEP = 2 };
int nbk_random(void* out, int32_t dtype, int64_t n, int32_t mode, float a, float b,
               const int64_t* state, uint32_t stream_id, void* stream);
int nbk_rng_advance(int64_t* state, void* stream);

/* ===================================================================== */
/*  Optimizer updates, all parameters in one launch                       */
/* ===================================================================== */
/* The reference updates a parameter pytree leaf by leaf with tensor arithmetic
 * (sgd_step nabla/nn/optim/functional.py:14-39, adamw_step 116-162, mapped over the leaves by
 * sgd_update 42-113 and adamw_update nabla/nn/optim/optimizer.py:242-305).  These two entry
 * points take the whole list: `tensors` is a host array of n entries, every entry the pointers of
 * one leaf -- all of them in `dtype` (NBK_F32 or NBK_BF16), contiguous, `numel` elements.  The
 * *_out pointers may be the inputs themselves (an in-place step) or fresh storage (the
 * functional form).  Arithmetic is fp32 in registers, one rounding per stored result.  One
 * launch per NBK_OPT_MULTI_MAX tensors. */
#define NBK_OPT_MULTI_MAX 48
typedef struct nbk_opt_tensor {
  const void* param; const void* grad;
  const void* m;        /* AdamW first moment / SGD momentum buffer (unused without momentum) */
  const void* v;        /* AdamW second moment (unused by SGD)                                 */
  void* param_out; void* m_out; void* v_out;
  int64_t numel;
} nbk_opt_tensor;
/* m' = beta1 m + (1-beta1) g;  v' = beta2 v + (1-beta2) g^2;
 * p' = p - lr ((m'/c1) / (sqrt(v'/c2) + eps) + weight_decay p)        (decoupled decay)
 * Bias corrections: with bias_correction == 0, c1 = c2 = 1.  Otherwise, when `step` is NULL the
 * host passes c1 = 1 - beta1^t and c2 = 1 - beta2^t; when `step` points to a device fp32 scalar
 * holding t (the counter is data inside a compiled step: optimizer.py:262-268), the kernel
 * computes c = 1 - exp(t log beta) itself from log_beta1 / log_beta2. */
typedef struct nbk_adamw_desc {
  float lr, beta1, beta2, eps, weight_decay;
  float c1, c2;
  float log_beta1, log_beta2;
  int32_t bias_correction;
  const float* step;
  int32_t dtype;
  int32_t reserved;
} nbk_adamw_desc;
int nbk_adamw_multi(const nbk_adamw_desc* d, const nbk_opt_tensor* tensors, int32_t n, void* stream);
/* dir = g + weight_decay p;  with momentum != 0: buf' = momentum buf + dir, dir = buf';
 * p' = p - lr dir.  (A leaf without a buffer yet passes zeros: the first step then adopts the
 * direction as the buffer, as functional.py:30-34 does.) */
typedef struct nbk_sgd_desc {
  float lr, momentum, weight_decay;
  int32_t dtype;
} nbk_sgd_desc;
int nbk_sgd_multi(const nbk_sgd_desc* d, const nbk_opt_tensor* tensors, int32_t n, void* stream);

/* ===================================================================== */
/*  Measurement helpers                                                   */
/* ===================================================================== */
/* HIP events on the caller's stream, so that bench code can time the very
 * stream the kernels run on. */
int nbk_event_create(void** ev);
int nbk_event_record(void* ev, void* stream);
int nbk_event_elapsed_ms(void* start, void* stop, float* ms); /* syncs stop */
int nbk_event_destroy(void* ev);
int nbk_stream_sync(void* stream);

/* ===================================================================== */
/*  Plan replay as a HIP graph                                            */
/* ===================================================================== */
/* The reference replays a compiled model once per step
 * (CompiledFunction._execute_cached_impl, nabla/transforms/compile.py:508-555);
 * here a cached plan is a fixed sequence of launches, and when a step runs again
 * on the same buffers the sequence is recorded once and replayed with a single
 * call.  Capture needs a stream of its own (the default stream cannot record):
 *   nbk_stream_create(&s); nbk_graph_begin_capture(s);
 *   ... every nbk_* launch of the plan with stream = s (nothing executes) ...
 *   nbk_graph_end_capture(s, &g);      then per step: nbk_graph_launch(g, any stream)
 * The recording holds the pointers it was made with; the caller replays only while
 * they are unchanged.  No memset nodes are ever recorded (nbk_fill is a kernel). */
int nbk_stream_create(void** stream);            /* non-blocking, default priority */
int nbk_stream_destroy(void* stream);
int nbk_graph_begin_capture(void* stream);
int nbk_graph_end_capture(void* stream, void** graph_exec);
int nbk_graph_launch(void* graph_exec, void* stream);
int nbk_graph_destroy(void* graph_exec);

#ifdef __cplusplus
}
#endif
#endif /* NBK_H_ */
