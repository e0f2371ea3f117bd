"""Row-program instruction set shared by the assembler, the HIP interpreter
(nabla_amd/csrc/rowprog.hip) and the numpy emulator used by the CPU tests.
Numbers must match ``enum nbk_rp_op`` in include/nbk.h (a test compares them).
"""
from __future__ import annotations

HALT, BODY, LDG, STG, LDR, STR, IMM, COLIDX, LEADIDX, ACCINIT, ACC, RED = range(12)

UNARY = {
    "mov": 16, "neg": 17, "relu": 18, "exp": 19, "log": 20, "sqrt": 21, "rsqrt": 22, "erf": 23,
    "gelu": 24, "tanh": 25, "sigmoid": 26, "abs": 27, "rbf16": 28, "not": 29, "trunc": 30,
    "nez": 31,
    "dgelu": 50, "sin": 51, "cos": 52,  # the block 16..31 is full
}
BINARY = {
    "add": 32, "sub": 33, "mul": 34, "div": 35, "max": 36, "min": 37, "gt": 38, "ge": 39,
    "eq": 40, "ne": 41, "lt": 42, "le": 43, "pow": 44, "and": 45, "or": 46,
}
TERNARY = {"where": 48, "fma": 49}
# int32 registers (values of int32 / int64 tensors); comparisons give a float 0 / 1
INT_BINARY = {"iadd": 64, "isub": 65, "imul": 66, "imax": 67, "imin": 68, "igt": 69, "ige": 70,
              "ieq": 71, "ine": 72, "ilt": 73, "ile": 74}
INT_UNARY = {"ineg": 80, "iabs": 81, "irelu": 82, "i2f": 83, "f2i": 84, "inez": 85}
UNARY.update(INT_UNARY)
BINARY.update(INT_BINARY)
#: float elementwise function -> its form on integer registers
INT_FORM = {"add": "iadd", "sub": "isub", "mul": "imul", "max": "imax", "min": "imin", "gt": "igt",
            "ge": "ige", "eq": "ieq", "ne": "ine", "lt": "ilt", "le": "ile", "neg": "ineg",
            "abs": "iabs", "relu": "irelu", "nez": "inez", "mov": "mov"}
#: elementwise functions of the 64-bit integer kernel (nbk_ew_int64), under their float codes
INT64_FNS = ("mov", "trunc", "neg", "abs", "relu", "not", "nez", "add", "sub", "mul", "div", "max", "min",
             "gt", "ge", "eq", "ne", "lt", "le", "pow", "and", "or", "where", "fma")
EW = {**UNARY, **BINARY, **TERNARY}
EW_NAME = {v: k for k, v in EW.items()}

RED_KIND = {"sum": 0, "max": 1, "min": 2}

MAX_OPERANDS = 20
MAX_INS = 224
MAX_IMM = 24
MAX_LEAD = 4
NVEC = 16
NSCL = 16
NACC = 4
MAX_STAGE = 4
STAGE_BYTES = 64 * 1024
MAX_BLOCK = 512

STRUCT_NAMES = {
    "HALT": HALT, "BODY": BODY, "LDG": LDG, "STG": STG, "LDR": LDR, "STR": STR, "IMM": IMM,
    "COLIDX": COLIDX, "LEADIDX": LEADIDX, "ACCINIT": ACCINIT, "ACC": ACC, "RED": RED,
}
