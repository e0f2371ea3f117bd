"""ctypes binding of libnbk.so (declarations in include/nbk.h).

There is no fallback: if the library is missing, or the ABI version differs,
loading raises.  Every entry point returns a status; non-zero becomes a Python
exception carrying ``nbk_last_error()`` (``ValueError`` for argument errors,
``RuntimeError`` otherwise) -- the reference surfaces MAX failures the same way
(nabla/ops/utils.py:574-575, tests/unit/FAILING_TESTS.md).
"""
from __future__ import annotations

import ctypes as C
from pathlib import Path

from . import isa

LIB_PATH = Path(__file__).resolve().parents[1] / "csrc" / "libnbk.so"
ABI_VERSION = 24

MAX_RANK = 8


class Operand(C.Structure):
    _fields_ = [
        ("ptr", C.c_void_p),
        ("lead_stride", C.c_int64 * isa.MAX_LEAD),
        ("col_stride", C.c_int32),
        ("dtype", C.c_int32),
        ("vec_ok", C.c_int32),
        ("stage_slot", C.c_int32),
    ]


class Ins(C.Structure):
    _fields_ = [
        ("op", C.c_uint8), ("dst", C.c_uint8), ("a", C.c_uint8), ("b", C.c_uint8),
        ("c", C.c_uint8), ("pad", C.c_uint8), ("aux", C.c_uint16),
    ]


class RowProg(C.Structure):
    _fields_ = [
        ("lead_dim", C.c_int64 * isa.MAX_LEAD),
        ("C", C.c_int64),
        ("n_lead", C.c_int32),
        ("n_operands", C.c_int32),
        ("n_ins", C.c_int32),
        ("n_imm", C.c_int32),
        ("has_reduce", C.c_int32),
        ("block", C.c_int32),
        ("n_stage", C.c_int32),
        ("reserved", C.c_int32),
        ("imm", C.c_float * isa.MAX_IMM),
        ("operand", Operand * isa.MAX_OPERANDS),
        ("ins", Ins * isa.MAX_INS),
    ]


class GemmTerm(C.Structure):
    _fields_ = [
        ("A", C.c_void_p), ("B", C.c_void_p),
        ("K", C.c_int64), ("a_rs", C.c_int64), ("a_cs", C.c_int64), ("b_rs", C.c_int64), ("b_cs", C.c_int64),
    ]


class GemmDesc(C.Structure):
    _fields_ = [
        ("A", C.c_void_p), ("B", C.c_void_p), ("C", C.c_void_p),
        ("bias", C.c_void_p), ("residual", C.c_void_p),
        ("M", C.c_int64), ("N", C.c_int64), ("K", C.c_int64),
        ("a_rs", C.c_int64), ("a_cs", C.c_int64), ("b_rs", C.c_int64), ("b_cs", C.c_int64),
        ("ldc", C.c_int64),
        ("batch", C.c_int64), ("a_bs", C.c_int64), ("b_bs", C.c_int64), ("c_bs", C.c_int64),
        ("batch_inner", C.c_int64), ("a_bs2", C.c_int64), ("b_bs2", C.c_int64), ("c_bs2", C.c_int64),
        ("dtype_ab", C.c_int32), ("dtype_c", C.c_int32),
        ("act", C.c_int32), ("batch_reduce", C.c_int32),
        ("alpha", C.c_float), ("residual_op", C.c_int32),
        ("C_aux", C.c_void_p), ("aux_op", C.c_int32), ("reserved", C.c_int32),
        ("colsum", C.c_void_p),
        ("n_terms", C.c_int32), ("reserved2", C.c_int32),
        ("term", GemmTerm * 4),
    ]


class GemmNf4Desc(C.Structure):
    _fields_ = [
        ("A", C.c_void_p), ("codes", C.c_void_p), ("scales", C.c_void_p), ("C", C.c_void_p),
        ("M", C.c_int64), ("w_rows", C.c_int64), ("w_cols", C.c_int64),
        ("lda", C.c_int64), ("ldc", C.c_int64),
        ("block", C.c_int32), ("transpose_w", C.c_int32), ("dtype", C.c_int32), ("alpha", C.c_float),
    ]


class ConvDesc(C.Structure):
    _fields_ = [
        ("N", C.c_int64), ("H", C.c_int64), ("W", C.c_int64), ("Cin", C.c_int64),
        ("R", C.c_int64), ("S", C.c_int64), ("Cout", C.c_int64), ("Ho", C.c_int64),
        ("Wo", C.c_int64),
        ("stride_h", C.c_int32), ("stride_w", C.c_int32),
        ("pad_t", C.c_int32), ("pad_b", C.c_int32), ("pad_l", C.c_int32), ("pad_r", C.c_int32),
        ("dtype", C.c_int32), ("act", C.c_int32),
    ]


class PoolDesc(C.Structure):
    _fields_ = [
        ("N", C.c_int64), ("H", C.c_int64), ("W", C.c_int64), ("C", C.c_int64),
        ("Ho", C.c_int64), ("Wo", C.c_int64),
        ("kh", C.c_int32), ("kw", C.c_int32), ("stride_h", C.c_int32), ("stride_w", C.c_int32),
        ("pad_t", C.c_int32), ("pad_l", C.c_int32),
        ("dtype", C.c_int32), ("reserved", C.c_int32),
    ]


class AttnDesc(C.Structure):
    _fields_ = [
        ("B", C.c_int64), ("H", C.c_int64), ("S", C.c_int64), ("hd", C.c_int64),
        ("scale", C.c_float), ("causal", C.c_int32), ("dtype", C.c_int32), ("reserved", C.c_int32),
    ]


class AttnTensor(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("sb", C.c_int64), ("ss", C.c_int64), ("sh", C.c_int64)]


class ReduceTask(C.Structure):
    _fields_ = [
        ("in_", C.c_void_p), ("out", C.c_void_p),
        ("outer", C.c_int64), ("red", C.c_int64), ("inner", C.c_int64),
        ("dtype_in", C.c_int32), ("dtype_out", C.c_int32), ("kind", C.c_int32), ("reserved", C.c_int32),
    ]


class OptTensor(C.Structure):
    _fields_ = [
        ("param", C.c_void_p), ("grad", C.c_void_p), ("m", C.c_void_p), ("v", C.c_void_p),
        ("param_out", C.c_void_p), ("m_out", C.c_void_p), ("v_out", C.c_void_p), ("numel", C.c_int64),
    ]


class AdamwDesc(C.Structure):
    _fields_ = [
        ("lr", C.c_float), ("beta1", C.c_float), ("beta2", C.c_float), ("eps", C.c_float),
        ("weight_decay", C.c_float), ("c1", C.c_float), ("c2", C.c_float),
        ("log_beta1", C.c_float), ("log_beta2", C.c_float), ("bias_correction", C.c_int32),
        ("step", C.c_void_p), ("dtype", C.c_int32), ("reserved", C.c_int32),
    ]


class SgdDesc(C.Structure):
    _fields_ = [("lr", C.c_float), ("momentum", C.c_float), ("weight_decay", C.c_float),
                ("dtype", C.c_int32)]


class TensorDesc(C.Structure):
    _fields_ = [
        ("ptr", C.c_void_p), ("dtype", C.c_int32), ("rank", C.c_int32),
        ("shape", C.c_int64 * MAX_RANK), ("stride", C.c_int64 * MAX_RANK),
    ]


_SIGNATURES = {
    "nbk_init": ([C.c_int], C.c_int),
    "nbk_last_error": ([], C.c_char_p),
    "nbk_abi_version": ([], C.c_int),
    "nbk_stream_create": ([C.POINTER(C.c_void_p)], C.c_int),
    "nbk_stream_destroy": ([C.c_void_p], C.c_int),
    "nbk_graph_begin_capture": ([C.c_void_p], C.c_int),
    "nbk_graph_end_capture": ([C.c_void_p, C.POINTER(C.c_void_p)], C.c_int),
    "nbk_graph_launch": ([C.c_void_p, C.c_void_p], C.c_int),
    "nbk_graph_destroy": ([C.c_void_p], C.c_int),
    "nbk_rowprog_launch": ([C.POINTER(RowProg), C.c_void_p], C.c_int),
    "nbk_rowprog_is_specialized": ([C.POINTER(RowProg)], C.c_int),
    "nbk_rowprog_hash": ([C.POINTER(RowProg)], C.c_uint64),
    "nbk_reduce_mid": ([C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_int64,
                        C.c_int64, C.c_int32, C.c_void_p], C.c_int),
    "nbk_random": ([C.c_void_p, C.c_int32, C.c_int64, C.c_int32, C.c_float, C.c_float, C.c_void_p,
                    C.c_uint32, C.c_void_p], C.c_int),
    "nbk_rng_advance": ([C.c_void_p, C.c_void_p], C.c_int),
    "nbk_adamw_multi": ([C.POINTER(AdamwDesc), C.POINTER(OptTensor), C.c_int32, C.c_void_p], C.c_int),
    "nbk_sgd_multi": ([C.POINTER(SgdDesc), C.POINTER(OptTensor), C.c_int32, C.c_void_p], C.c_int),
    "nbk_reduce_mid_batch": ([C.POINTER(ReduceTask), C.c_int32, C.c_void_p], C.c_int),
    "nbk_copy_strided": ([C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                          C.POINTER(C.c_int64), C.POINTER(C.c_int64), C.POINTER(C.c_int64),
                          C.c_void_p], C.c_int),
    "nbk_fill": ([C.c_void_p, C.c_int32, C.c_int64, C.c_double, C.c_void_p], C.c_int),
    "nbk_gemm": ([C.POINTER(GemmDesc), C.c_void_p], C.c_int),
    "nbk_gemm_nf4": ([C.POINTER(GemmNf4Desc), C.c_void_p], C.c_int),
    "nbk_conv2d_fwd": ([C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                        C.c_void_p], C.c_int),
    "nbk_conv2d_dgrad": ([C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p],
                         C.c_int),
    "nbk_conv2d_wgrad_workspace": ([C.POINTER(ConvDesc)], C.c_int64),
    "nbk_conv2d_wgrad": ([C.POINTER(ConvDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                          C.c_int64, C.c_void_p], C.c_int),
    "nbk_maxpool2d_fwd": ([C.POINTER(PoolDesc), C.c_void_p, C.c_void_p, C.c_void_p], C.c_int),
    "nbk_maxpool2d_bwd": ([C.POINTER(PoolDesc), C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                           C.c_void_p], C.c_int),
    "nbk_avgpool2d_fwd": ([C.POINTER(PoolDesc), C.c_void_p, C.c_void_p, C.c_void_p], C.c_int),
    "nbk_avgpool2d_bwd": ([C.POINTER(PoolDesc), C.c_void_p, C.c_void_p, C.c_void_p], C.c_int),
    "nbk_attention_fwd": ([C.POINTER(AttnDesc)] + [C.POINTER(AttnTensor)] * 5 + [C.c_void_p, C.c_void_p],
                          C.c_int),
    "nbk_attention_bwd_workspace": ([C.POINTER(AttnDesc)], C.c_int64),
    "nbk_attention_bwd": ([C.POINTER(AttnDesc)] + [C.POINTER(AttnTensor)] * 5 + [C.c_void_p] +
                          [C.POINTER(AttnTensor)] * 4 + [C.c_void_p, C.c_int64, C.c_void_p], C.c_int),
    "nbk_attention_bwd_static": ([C.POINTER(AttnDesc)] + [C.POINTER(AttnTensor)] * 5 + [C.c_void_p] +
                                 [C.POINTER(AttnTensor)] * 4 + [C.c_void_p], C.c_int),
    "nbk_gather": ([C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64,
                    C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p], C.c_int),
    "nbk_scatter": ([C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int64, C.c_int64,
                     C.c_int64, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p], C.c_int),
    "nbk_argmax_rows": ([C.c_void_p, C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int32,
                         C.c_void_p], C.c_int),
    "nbk_custom": ([C.c_char_p, C.c_char_p, C.POINTER(TensorDesc), C.c_int,
                    C.POINTER(TensorDesc), C.c_int, C.c_void_p], C.c_int),
    "nbk_ew_int64": ([C.c_int32, C.POINTER(TensorDesc), C.POINTER(C.c_int64), C.c_int32,
                      C.POINTER(TensorDesc), C.c_void_p], C.c_int),
    "nbk_event_create": ([C.POINTER(C.c_void_p)], C.c_int),
    "nbk_event_record": ([C.c_void_p, C.c_void_p], C.c_int),
    "nbk_event_elapsed_ms": ([C.c_void_p, C.c_void_p, C.POINTER(C.c_float)], C.c_int),
    "nbk_event_destroy": ([C.c_void_p], C.c_int),
    "nbk_stream_sync": ([C.c_void_p], C.c_int),
}

EXPORTS = tuple(_SIGNATURES)

_lib = None


class NbkError(RuntimeError):
    pass


def load(path: Path | None = None):
    """Load libnbk.so; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    p = Path(path) if path else LIB_PATH
    if not p.exists():
        raise NbkError(
            f"{p} is missing: build it with `python -m nabla_amd.backend.build` "
            "(there is no CPU fallback for the kernel library)"
        )
    lib = C.CDLL(str(p))
    for name, (argtypes, restype) in _SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.argtypes = argtypes
        fn.restype = restype
    got = lib.nbk_abi_version()
    if got != ABI_VERSION:
        raise NbkError(f"{p} has ABI version {got}, the Python shim expects {ABI_VERSION}")
    _lib = lib
    return lib


def check(rc: int) -> None:
    if rc == 0:
        return
    msg = load().nbk_last_error().decode("utf-8", "replace")
    if rc == -1:
        raise ValueError(msg)
    raise RuntimeError(msg)
