"""TEST INFRASTRUCTURE -- not part of the product.

A numpy/torch-CPU interpreter of the launch records that the lowering pass
produces (row programs, strided copies, GEMM / conv / pool / gather records).
It exists so that the host-side logic -- tracing, autodiff replay, fusion,
view folding, register allocation, buffer planning -- can be checked on a
machine without a GPU, and so that the HIP interpreter can be compared with a
second implementation of the same instruction set.  Only tests may install it
(``nabla_amd.backend.executor.set_executor``); the package itself never does.
"""
from __future__ import annotations

import numpy as np
import torch
from scipy import special as _sp

from nabla_amd.backend import isa
from nabla_amd.backend.planner import Plan, ViewRef
from nabla_amd.core.dtype import DType

_F32 = np.float32


def _round_bf16(a: np.ndarray) -> np.ndarray:
    t = torch.from_numpy(np.ascontiguousarray(a.astype(np.float32)))
    return t.to(torch.bfloat16).to(torch.float32).numpy()


_UNARY = {
    "mov": lambda a: a,
    "neg": lambda a: -a,
    "relu": lambda a: np.maximum(a, _F32(0)),
    "exp": lambda a: np.exp(a),
    "log": lambda a: np.log(a),
    "sqrt": lambda a: np.sqrt(a),
    "rsqrt": lambda a: (_F32(1) / np.sqrt(a)).astype(_F32),
    "erf": lambda a: _sp.erf(a.astype(np.float64)).astype(_F32),
    "gelu": lambda a: (0.5 * a.astype(np.float64) * (1.0 + _sp.erf(a.astype(np.float64) / np.sqrt(2.0)))).astype(_F32),
    "dgelu": lambda a: (0.5 * (1.0 + _sp.erf(a.astype(np.float64) / np.sqrt(2.0))) +
                        a.astype(np.float64) * np.exp(-0.5 * a.astype(np.float64) ** 2) / np.sqrt(2.0 * np.pi)).astype(_F32),
    "tanh": lambda a: np.tanh(a),
    "sin": lambda a: np.sin(a),
    "cos": lambda a: np.cos(a),
    "sigmoid": lambda a: (_F32(1) / (_F32(1) + np.exp(-a))).astype(_F32),
    "abs": lambda a: np.abs(a),
    "rbf16": _round_bf16,
    "not": lambda a: (a == 0).astype(_F32),
    "trunc": lambda a: np.trunc(a),
    "nez": lambda a: (a != 0).astype(_F32),
}
_BINARY = {
    "add": lambda a, b: a + b,
    "sub": lambda a, b: a - b,
    "mul": lambda a, b: a * b,
    "div": lambda a, b: a / b,
    "max": lambda a, b: np.maximum(a, b),
    "min": lambda a, b: np.minimum(a, b),
    "gt": lambda a, b: (a > b).astype(_F32),
    "ge": lambda a, b: (a >= b).astype(_F32),
    "eq": lambda a, b: (a == b).astype(_F32),
    "ne": lambda a, b: (a != b).astype(_F32),
    "lt": lambda a, b: (a < b).astype(_F32),
    "le": lambda a, b: (a <= b).astype(_F32),
    "pow": lambda a, b: np.power(a, b),
    "and": lambda a, b: ((a != 0) & (b != 0)).astype(_F32),
    "or": lambda a, b: ((a != 0) | (b != 0)).astype(_F32),
}


# Integer registers: values of int32 / int64 tensors are held as int32 in the 32 bits of a
# register (here: in the bytes of a float32 array) and computed with the integer forms below.
_I32 = np.int32


def _ibits(a) -> np.ndarray:
    """float32 array -> the int32 values its bytes hold."""
    return np.ascontiguousarray(a, dtype=_F32).view(_I32)


def _fbits(i) -> np.ndarray:
    """int values (wrapped to int32) -> float32 array with those bytes."""
    return np.ascontiguousarray(np.asarray(i).astype(_I32)).view(_F32)


_UNARY.update({
    "ineg": lambda a: _fbits(-_ibits(a)),
    "iabs": lambda a: _fbits(np.abs(_ibits(a))),
    "irelu": lambda a: _fbits(np.maximum(_ibits(a), 0)),
    "i2f": lambda a: _ibits(a).astype(_F32),
    "f2i": lambda a: _fbits(np.trunc(np.nan_to_num(a.astype(np.float64))).clip(-2.0 ** 31, 2.0 ** 31 - 1)
                            .astype(np.int64)),
    "inez": lambda a: (_ibits(a) != 0).astype(_F32),
})
_BINARY.update({
    "iadd": lambda a, b: _fbits(_ibits(a).astype(np.int64) + _ibits(b)),
    "isub": lambda a, b: _fbits(_ibits(a).astype(np.int64) - _ibits(b)),
    "imul": lambda a, b: _fbits(_ibits(a).astype(np.int64) * _ibits(b)),
    "imax": lambda a, b: _fbits(np.maximum(_ibits(a), _ibits(b))),
    "imin": lambda a, b: _fbits(np.minimum(_ibits(a), _ibits(b))),
    "igt": lambda a, b: (_ibits(a) > _ibits(b)).astype(_F32),
    "ige": lambda a, b: (_ibits(a) >= _ibits(b)).astype(_F32),
    "ieq": lambda a, b: (_ibits(a) == _ibits(b)).astype(_F32),
    "ine": lambda a, b: (_ibits(a) != _ibits(b)).astype(_F32),
    "ilt": lambda a, b: (_ibits(a) < _ibits(b)).astype(_F32),
    "ile": lambda a, b: (_ibits(a) <= _ibits(b)).astype(_F32),
})


def _load_reg(t: torch.Tensor) -> np.ndarray:
    """Elements of an operand as register contents (int64 storage saturates to the int32 range)."""
    if t.dtype == torch.int64:
        return _fbits(np.clip(t.numpy(), -2 ** 31, 2 ** 31 - 1))
    if t.dtype == torch.int32:
        return _fbits(t.numpy())
    return _as_f32(t)


def _as_f32(t: torch.Tensor) -> np.ndarray:
    if t.dtype == torch.bfloat16 or t.dtype == torch.float16:
        return t.float().numpy()
    if t.dtype == torch.bool:
        return t.numpy().astype(_F32)
    return t.numpy().astype(_F32)


def _store(flat: torch.Tensor, idx: np.ndarray, vals: np.ndarray) -> None:
    """flat[idx] = vals with the destination's rounding."""
    if flat.dtype in (torch.int32, torch.int64):  # an integer register: its bits are the value
        v = torch.from_numpy(_ibits(vals).copy()).to(flat.dtype)
        flat[torch.from_numpy(idx.reshape(-1))] = v.reshape(-1)
        return
    v = torch.from_numpy(np.ascontiguousarray(vals.astype(_F32)))
    if flat.dtype == torch.bool:
        v = v != 0
    else:
        v = v.to(flat.dtype)
    flat[torch.from_numpy(idx.reshape(-1))] = v.reshape(-1)


def _ew_int64(a: dict, mem: list[torch.Tensor]) -> None:
    """The 64-bit integer elementwise kernel: operands widen to int64 (floats are cut toward
    zero), the arithmetic wraps modulo 2^64, division rounds toward zero."""
    dst = _view(mem, a["dst"])

    def widen(o):
        if isinstance(o, int):
            return np.int64(o)
        t = _view(mem, o)
        if t.dtype.is_floating_point:
            x = np.nan_to_num(np.trunc(t.double().numpy()), nan=0.0)
            return np.clip(x, -2.0 ** 63, 2.0 ** 63 - 1025).astype(np.int64)
        return t.numpy().astype(np.int64)

    def div(p, q):
        safe = np.where(q == 0, 1, q)
        r = np.abs(p) // np.abs(safe) * np.sign(p) * np.sign(safe)
        return np.where(q == 0, 0, r).astype(np.int64)

    def ipow(b, e):
        b, e = np.broadcast_arrays(np.asarray(b, np.int64), np.asarray(e, np.int64))
        out = np.empty(b.shape, np.int64)
        for idx in np.ndindex(b.shape):
            bb, ee = int(b[idx]), int(e[idx])
            if ee < 0:
                v = 1 if bb == 1 else ((-1 if ee & 1 else 1) if bb == -1 else 0)
            else:
                v = pow(bb, ee, 2 ** 64)
                v = v - 2 ** 64 if v >= 2 ** 63 else v
            out[idx] = v
        return out

    xs = [widen(o) for o in a["operands"]]
    fn = a["fn"]
    with np.errstate(over="ignore"):
        r = {
            "mov": lambda p: p, "trunc": lambda p: p, "neg": lambda p: -p, "abs": lambda p: np.abs(p),
            "relu": lambda p: np.maximum(p, 0), "not": lambda p: p == 0, "nez": lambda p: p != 0,
            "add": lambda p, q: p + q, "sub": lambda p, q: p - q, "mul": lambda p, q: p * q, "div": div,
            "max": np.maximum, "min": np.minimum, "gt": lambda p, q: p > q, "ge": lambda p, q: p >= q,
            "eq": lambda p, q: p == q, "ne": lambda p, q: p != q, "lt": lambda p, q: p < q,
            "le": lambda p, q: p <= q, "pow": ipow, "and": lambda p, q: (p != 0) & (q != 0),
            "or": lambda p, q: (p != 0) | (q != 0), "where": lambda c, p, q: np.where(c != 0, p, q),
            "fma": lambda p, q, c: p * q + c,
        }[fn](*xs)
    r = np.broadcast_to(np.asarray(r), tuple(dst.shape)).astype(np.int64)
    if dst.dtype == torch.bool:
        dst.copy_(torch.from_numpy(r != 0))
    elif dst.dtype == torch.int32:
        dst.copy_(torch.from_numpy(r.astype(np.int32)))
    elif dst.dtype == torch.int64:
        dst.copy_(torch.from_numpy(r.copy()))
    else:
        dst.copy_(torch.from_numpy(r.astype(np.float32)).to(dst.dtype))


def run_rowprog(a: dict, mem: list[torch.Tensor]) -> None:
    lead, C = a["lead"], a["C"]
    R = int(np.prod(lead)) if lead else 1
    ops = a["operands"]
    imm = a["imm"]
    # per-row leading indices
    lead_idx = np.stack(np.unravel_index(np.arange(R), lead), axis=0) if lead else np.zeros((0, R), np.int64)

    def row_off(o):
        off = np.full(R, o.offset, dtype=np.int64)
        for k, s in enumerate(o.lead_strides):
            off = off + lead_idx[k].astype(np.int64) * s
        return off

    cols = np.arange(C, dtype=np.int64)
    V = {}
    S = {}
    ACC = {}
    ins = a["ins"]

    def rd(r):
        if r < isa.NVEC:
            return V[r]
        return S[r][:, None]

    def rs(r):
        return S[r]

    pc = 0
    while pc < len(ins):
        op, dst, x, y, z, aux = ins[pc]
        if op == isa.HALT:
            break
        if op == isa.BODY:
            for q in range(pc + 1, pc + 1 + aux):
                bop, bd, bx, by, bz, _ = ins[q]
                if bop == isa.LDG:
                    o = ops[bx]
                    idx = row_off(o)[:, None] + cols[None, :] * o.col_stride
                    V[bd] = _load_reg(mem[o.buf][torch.from_numpy(idx.reshape(-1))]).reshape(R, C)
                elif bop == isa.STG:
                    o = ops[bd]
                    idx = row_off(o)[:, None] + cols[None, :] * o.col_stride
                    _store(mem[o.buf], idx, np.broadcast_to(rd(bx), (R, C)))
                elif bop == isa.ACC:
                    v = np.broadcast_to(rd(bx), (R, C)).astype(_F32)
                    red = {0: np.sum, 1: np.max, 2: np.min}[by]
                    part = red(v, axis=1).astype(_F32)
                    ACC[bd] = {0: np.add, 1: np.maximum, 2: np.minimum}[by](ACC[bd], part).astype(_F32)
                elif bop == isa.COLIDX:
                    as_reg = _fbits(cols) if bx else cols.astype(_F32)
                    V[bd] = np.broadcast_to(as_reg[None, :], (R, C)).copy()
                elif bop in isa.EW_NAME:
                    name = isa.EW_NAME[bop]
                    with np.errstate(all="ignore"):
                        if name in _UNARY:
                            r = _UNARY[name](np.broadcast_to(rd(bx), (R, C)).astype(_F32))
                        elif name in _BINARY:
                            r = _BINARY[name](rd(bx).astype(_F32), rd(by).astype(_F32))
                        elif name == "where":
                            r = _fbits(np.where(rd(bx) != 0, _ibits(rd(by)), _ibits(rd(bz))))  # moves bits
                        else:  # fma
                            r = (rd(bx).astype(np.float64) * rd(by) + rd(bz))
                    V[bd] = np.broadcast_to(np.asarray(r, dtype=_F32), (R, C)).copy()
                else:
                    raise AssertionError(f"opcode {bop} in a body")
            pc += 1 + aux
            continue
        if op == isa.IMM:
            S[dst] = _fbits(np.full(R, imm[x])) if isinstance(imm[x], int) else np.full(R, imm[x], dtype=_F32)
        elif op == isa.LDR:
            o = ops[x]
            S[dst] = _load_reg(mem[o.buf][torch.from_numpy(row_off(o))])
        elif op == isa.STR:
            o = ops[dst]
            _store(mem[o.buf], row_off(o), rs(x))
        elif op == isa.LEADIDX:
            S[dst] = _fbits(lead_idx[x]) if y else lead_idx[x].astype(_F32)
        elif op == isa.ACCINIT:
            ACC[dst] = np.full(R, {0: 0.0, 1: -np.inf, 2: np.inf}[x], dtype=_F32)
        elif op == isa.RED:
            S[dst] = ACC[x].astype(_F32)
        elif op in isa.EW_NAME:
            name = isa.EW_NAME[op]
            with np.errstate(all="ignore"):
                if name in _UNARY:
                    S[dst] = np.asarray(_UNARY[name](rs(x)), dtype=_F32)
                elif name in _BINARY:
                    S[dst] = np.asarray(_BINARY[name](rs(x), rs(y)), dtype=_F32)
                elif name == "where":
                    S[dst] = _fbits(np.where(rs(x) != 0, _ibits(rs(y)), _ibits(rs(z))))
                else:
                    S[dst] = (rs(x).astype(np.float64) * rs(y) + rs(z)).astype(_F32)
        else:
            raise AssertionError(f"opcode {op} in a prologue")
        pc += 1


def _view(mem, ref: ViewRef) -> torch.Tensor:
    return torch.as_strided(mem[ref.buf], ref.shape, ref.strides, ref.offset)


def _gemm(a, mem):
    bi = max(1, a.get("batch_inner", 1))
    bo = a["batch"] // bi

    def mat(ref, bs, bs2, rs, cs, rows, cols):
        base = mem[ref.buf]
        return torch.as_strided(base, (bo, bi, rows, cols), (bs, bs2 if bi > 1 else 0, rs, cs), ref.offset)
    A = mat(a["a"], a["a_bs"], a.get("a_bs2", 0), a["a_rs"], a["a_cs"], a["M"], a["K"]).float()
    B = mat(a["b"], a["b_bs"], a.get("b_bs2", 0), a["b_rs"], a["b_cs"], a["K"], a["N"]).float()
    prod = torch.matmul(A.double(), B.double())
    for t in a.get("terms") or ():  # more operand pairs in the same accumulator (batch 1)
        At = torch.as_strided(mem[t["a"].buf], (a["M"], t["K"]), (t["a_rs"], t["a_cs"]), t["a"].offset)
        Bt = torch.as_strided(mem[t["b"].buf], (t["K"], a["N"]), (t["b_rs"], t["b_cs"]), t["b"].offset)
        prod = prod + torch.matmul(At.double(), Bt.double())
    C = prod.float() * a.get("alpha", 1.0)
    if a.get("bias") is not None:  # added before the result is rounded, as in the kernel's epilogue
        C = C + _view(mem, a["bias"]).reshape(-1).float()
    if a.get("act") is not None:
        x = C.double()
        if a["act"] == "gelu":
            cdf = 0.5 * (1.0 + torch.erf(x / 2.0 ** 0.5))
            act, dact = x * cdf, cdf + x * torch.exp(-0.5 * x * x) / (2.0 * torch.pi) ** 0.5
        else:
            act, dact = torch.relu(x), (x > 0).double()
        if a.get("aux_dst") is not None:
            aux = mat(a["aux_dst"], a["c_bs"], a.get("c_bs2", 0), a["ldc"], 1, a["M"], a["N"])
            aux.copy_(dact.to(aux.dtype))
        C = act.float()
    if a.get("residual") is not None:
        res = a["residual"]
        R = mat(res, a["c_bs"], a.get("c_bs2", 0), a["ldc"], 1, a["M"], a["N"]).float()
        C = C * R if a["res_op"] == "mul" else C + R
    dst = a["dst"]
    out = mat(dst, a["c_bs"], a.get("c_bs2", 0), a["ldc"], 1, a["M"], a["N"])
    out.copy_(C.to(out.dtype))
    if a.get("colsum") is not None:  # sum over k of B, one row per batch slice, in C's dtype
        cs = _view(mem, a["colsum"]).reshape(a["batch"], a["N"])
        cs.copy_(B.double().sum(dim=2).reshape(a["batch"], a["N"]).to(cs.dtype))


_NF4_LEVELS = torch.tensor([-1.0, -0.6962, -0.5251, -0.3949, -0.2844, -0.1848, -0.0911, 0.0, 0.0796,
                            0.1609, 0.2461, 0.3379, 0.4407, 0.5626, 0.7230, 1.0], dtype=torch.float32)


def _gemm_nf4(a, mem):
    codes = _view(mem, a["codes"]).reshape(-1).long()
    scales = _view(mem, a["scales"]).reshape(-1).float()
    w = (_NF4_LEVELS[codes].reshape(-1, a["block"]) * scales[:, None]).reshape(a["w_shape"])
    dst = _view(mem, a["dst"])
    if dst.dtype == torch.bfloat16:  # level * scale is rounded to bf16 once, as in the kernel
        w = w.to(torch.bfloat16).float()
    x = _view(mem, a["x"]).reshape(a["M"], a["K"]).double()
    w = w.double().t() if a["transpose"] else w.double()
    dst.copy_((x @ w).reshape(dst.shape).to(dst.dtype))


def _update_list(kind, a, mem):
    """Optimizer step over a list of parameters, in float64 from the stored values
    (nabla/nn/optim/functional.py:14-39 and 116-162)."""
    for e in a["entries"]:
        ins = [_view(mem, r).double() for r in e["ins"]]
        outs = [_view(mem, r) for r in e["outs"]]
        p, g = ins[0], ins[1]
        if kind == "adamw_multi":
            m, v = ins[2], ins[3]
            b1, b2 = a["beta1"], a["beta2"]
            step = a["step"] if a["step"] is not None else float(_view(mem, a["step_ref"]).reshape(-1)[0])
            c1 = 1.0 - b1 ** step if a["bias_correction"] else 1.0
            c2 = 1.0 - b2 ** step if a["bias_correction"] else 1.0
            m_t = m * b1 + g * (1.0 - b1)
            v_t = v * b2 + g * g * (1.0 - b2)
            upd = (m_t / c1) / ((v_t / c2).sqrt() + a["eps"]) + p * a["weight_decay"]
            results = [p - upd * a["lr"], m_t, v_t]
        else:
            direction = g + p * a["weight_decay"]
            results = []
            if a["momentum"] != 0.0:
                direction = ins[2] * a["momentum"] + direction
                results = [direction]
            results.insert(0, p - direction * a["lr"])
        for dst, val in zip(outs, results):
            dst.copy_(val.to(dst.dtype))


def _conv(kind, a, mem):
    import torch.nn.functional as F
    pt, pb, pl, pr = a["padding"]
    sh, sw = a["stride"]
    ins = [_view(mem, r).float() for r in a["ins"]]
    dst = _view(mem, a["dst"])
    if kind == "conv2d":
        x, w = ins[0], ins[1]
        xp = F.pad(x.permute(0, 3, 1, 2), (pl, pr, pt, pb))
        y = F.conv2d(xp.double(), w.permute(3, 2, 0, 1).double(), stride=(sh, sw)).float()
        y = y.permute(0, 2, 3, 1)
        if a["has_bias"]:
            y = y + ins[2]
        if a.get("act") == "relu":  # the activation the planner folded into the launch
            y = torch.relu(y)
        dst.copy_(y.to(dst.dtype))
        return
    xs, ws = a["x_shape"], a["w_shape"]
    x = (ins[0] if kind == "conv2d_wgrad" else torch.zeros(xs)).double().requires_grad_(True)
    w = (ins[1] if kind == "conv2d_dgrad" else torch.zeros(ws)).double().requires_grad_(True)
    dy = (ins[0] if kind == "conv2d_dgrad" else ins[1]).double()
    xp = F.pad(x.permute(0, 3, 1, 2), (pl, pr, pt, pb))
    y = F.conv2d(xp, w.permute(3, 2, 0, 1), stride=(sh, sw)).permute(0, 2, 3, 1)
    (g,) = torch.autograd.grad(y, x if kind == "conv2d_dgrad" else w, dy)
    dst.copy_(g.float().to(dst.dtype))


def _pool(kind, a, mem):
    kh, kw = a["kernel"]
    sh, sw = a["stride"]
    pt, _, pl, _ = a["padding"]
    x = _view(mem, a["ins"][0]).float().numpy()
    N, H, W, C = x.shape
    _, Ho, Wo, _ = a["y_shape"]
    dst = _view(mem, a["dst"])
    if kind == "maxpool2d":
        y = np.full((N, Ho, Wo, C), -np.inf, dtype=_F32)
        for i in range(Ho):
            for j in range(Wo):
                h0, h1 = max(0, i * sh - pt), min(H, i * sh - pt + kh)
                w0, w1 = max(0, j * sw - pl), min(W, j * sw - pl + kw)
                if h0 < h1 and w0 < w1:
                    y[:, i, j, :] = x[:, h0:h1, w0:w1, :].max(axis=(1, 2))
        dst.copy_(torch.from_numpy(y).to(dst.dtype))
        return
    y = _view(mem, a["ins"][1]).float().numpy()
    dy = _view(mem, a["ins"][2]).float().numpy()
    dx = np.zeros_like(x)
    for i in range(Ho):
        for j in range(Wo):
            h0, h1 = max(0, i * sh - pt), min(H, i * sh - pt + kh)
            w0, w1 = max(0, j * sw - pl), min(W, j * sw - pl + kw)
            if h0 < h1 and w0 < w1:
                win = x[:, h0:h1, w0:w1, :]
                mask = (win == y[:, i:i + 1, j:j + 1, :]).astype(_F32)
                dx[:, h0:h1, w0:w1, :] += mask * dy[:, i:i + 1, j:j + 1, :]
    dst.copy_(torch.from_numpy(dx).to(dst.dtype))


def _attention(kind, a, mem):
    """Plain softmax attention in float64 on [B, H, S, hd] views; the backward through
    autograd of that same expression."""
    q, k, v = (_view(mem, a[n]).double() for n in ("q", "k", "v"))
    S = a["S"]

    def forward(q, k, v):
        s = (q @ k.transpose(-1, -2)) * a["scale"]
        if a["causal"]:
            keep = torch.ones(S, S, dtype=torch.bool).tril()
            s = s.masked_fill(~keep, float("-inf"))
        return torch.softmax(s, dim=-1) @ v, torch.logsumexp(s, dim=-1)

    if kind == "attention":
        o, lse = forward(q, k, v)
        dst = _view(mem, a["o"])
        dst.copy_(o.float().to(dst.dtype))
        _view(mem, a["lse"]).copy_(lse.float())
        if a.get("o_lo") is not None:  # what the rounding of o cut off, rounded the same way
            lo = _view(mem, a["o_lo"])
            lo.copy_((o.float() - dst.float()).to(lo.dtype))
        return
    q, k, v = (t.clone().requires_grad_(True) for t in (q, k, v))
    o, _ = forward(q, k, v)
    grads = torch.autograd.grad(o, (q, k, v), _view(mem, a["dout"]).double())
    for name, g in zip(("dq", "dk", "dv"), grads):
        dst = _view(mem, a[name])
        dst.copy_(g.float().to(dst.dtype))


def _avgpool(kind, a, mem):
    """Zero padding, window sums divided by kh * kw; the backward is its transpose."""
    kh, kw = a["kernel"]
    sh, sw = a["stride"]
    pt, _, pl, _ = a["padding"]
    N, H, W, C = a["x_shape"]
    _, Ho, Wo, _ = a["y_shape"]
    src = _view(mem, a["ins"][0]).double().numpy()
    dst = _view(mem, a["dst"])
    res = np.zeros((N, Ho, Wo, C) if kind == "avgpool2d" else (N, H, W, C))
    for i in range(Ho):
        for j in range(Wo):
            h0, h1 = max(0, i * sh - pt), min(H, i * sh - pt + kh)
            w0, w1 = max(0, j * sw - pl), min(W, j * sw - pl + kw)
            if h0 >= h1 or w0 >= w1:
                continue
            if kind == "avgpool2d":
                res[:, i, j, :] = src[:, h0:h1, w0:w1, :].sum(axis=(1, 2)) / (kh * kw)
            else:
                res[:, h0:h1, w0:w1, :] += src[:, i:i + 1, j:j + 1, :] / (kh * kw)
    dst.copy_(torch.from_numpy(res).float().to(dst.dtype))


class EmulatedPlan:
    def __init__(self, plan: Plan, rng_state: list | None = None):
        self.plan = plan
        self.rng_state = rng_state if rng_state is not None else [0, 0]  # [seed, runs], shared

    def run(self, inputs):
        plan = self.plan
        mem: list = [None] * len(plan.bufs)
        outs = [None] * len(plan.outputs)
        for b in plan.bufs:
            if b.role == "input":
                mem[b.id] = inputs[b.index].contiguous().reshape(-1)
            else:
                # poison temporaries so that reads of unwritten memory show up
                t = torch.empty(max(b.numel, 1), dtype=b.dtype.to_torch())
                if t.dtype.is_floating_point:
                    t.fill_(float("nan"))
                else:
                    t.zero_()
                mem[b.id] = t
        for st in plan.steps:
            a, k = st.attrs, st.kind
            if k == "rowprog":
                run_rowprog(a, mem)
            elif k == "copy":
                src = _view(mem, a["src"])
                dst = _view(mem, a["dst"])
                dst.copy_(src.to(dst.dtype))
            elif k == "fill":
                v = a["value"]
                t = mem[a["buf"]]
                t.fill_(bool(v) if t.dtype == torch.bool else (int(v) if not t.dtype.is_floating_point else v))
            elif k in ("reduce_mid", "reduce_batch"):
                for t in ([a] if k == "reduce_mid" else a["tasks"]):
                    src = mem[t["src"].buf][t["src"].offset:t["src"].offset + t["outer"] * t["red"] * t["inner"]]
                    if src.dtype in (torch.int32, torch.int64):  # exact, 64-bit accumulator
                        xi = src.numpy().astype(np.int64).reshape(t["outer"], t["red"], t["inner"])
                        ri = {"sum": xi.sum(axis=1), "max": xi.max(axis=1), "min": xi.min(axis=1)}[t["fn"]]
                        d = t["dst"]
                        flat = mem[d.buf]
                        vals = torch.from_numpy(ri.reshape(-1))
                        flat[d.offset:d.offset + vals.numel()] = vals.to(flat.dtype)
                        continue
                    x = _as_f32(src).reshape(t["outer"], t["red"], t["inner"])
                    r = {"sum": x.sum(axis=1, dtype=np.float64), "max": x.max(axis=1), "min": x.min(axis=1)}[t["fn"]]
                    d = t["dst"]
                    _store(mem[d.buf], d.offset + np.arange(t["outer"] * t["inner"]), np.asarray(r, dtype=_F32))
            elif k == "gemm":
                _gemm(a, mem)
            elif k == "gemm_nf4":
                _gemm_nf4(a, mem)
            elif k in ("adamw_multi", "sgd_multi"):
                _update_list(k, a, mem)
            elif k == "random":
                from . import philox
                seed, run = self.rng_state
                n = a["numel"]
                vals = {"uniform": lambda: philox.uniform(n, a["a"], a["b"], seed, run, a["stream"]),
                        "normal": lambda: philox.normal(n, a["a"], a["b"], seed, run, a["stream"]),
                        "keep": lambda: philox.keep_mask(n, a["a"], seed, run, a["stream"])}[a["mode"]]()
                dst = _view(mem, a["dst"])
                dst.copy_(torch.from_numpy(np.ascontiguousarray(vals)).reshape(dst.shape).to(dst.dtype))
            elif k == "rng_advance":
                self.rng_state[1] += 1
            elif k in ("conv2d", "conv2d_dgrad", "conv2d_wgrad"):
                _conv(k, a, mem)
            elif k in ("maxpool2d", "maxpool2d_bwd"):
                _pool(k, a, mem)
            elif k in ("avgpool2d", "avgpool2d_bwd"):
                _avgpool(k, a, mem)
            elif k in ("attention", "attention_bwd"):
                _attention(k, a, mem)
            elif k == "gather":
                t = _view(mem, a["table"]).reshape(a["outer"], a["axis_len"], a["inner"])
                ix = _view(mem, a["idx"]).reshape(-1).long()
                if bool(((ix < -a["axis_len"]) | (ix >= a["axis_len"])).any()):
                    raise IndexError("gather: index out of range")
                ix = torch.where(ix < 0, ix + a["axis_len"], ix)
                _view(mem, a["dst"]).copy_(t.index_select(1, ix).reshape(a["dst"].shape))
            elif k == "scatter":
                dst = _view(mem, a["dst"]).reshape(a["outer"], a["axis_len"], a["inner"])
                up = _view(mem, a["upd"]).reshape(a["outer"], a["n_idx"], a["inner"])
                ix = _view(mem, a["idx"]).reshape(-1).long()
                if bool(((ix < -a["axis_len"]) | (ix >= a["axis_len"])).any()):
                    raise IndexError("scatter: index out of range")
                ix = torch.where(ix < 0, ix + a["axis_len"], ix)
                for j in range(a["n_idx"]):  # in order: the last write to a row wins
                    dst[:, int(ix[j]), :] = up[:, j, :]
            elif k == "ew64":
                _ew_int64(a, mem)
            elif k == "argreduce":
                src = _view(mem, a["src"])
                if src.dtype in (torch.int32, torch.int64):  # integers compare exactly
                    xi = src.numpy().astype(np.int64).reshape(a["rows"], a["C"])
                    r = np.argmin(xi, axis=1) if a["fn"] == "min" else np.argmax(xi, axis=1)
                    _view(mem, a["dst"]).copy_(torch.from_numpy(r.astype(np.int64)).reshape(a["dst"].shape))
                    continue
                x = _as_f32(_view(mem, a["src"])).reshape(a["rows"], a["C"])
                r = np.argmin(x, axis=1) if a["fn"] == "min" else np.argmax(x, axis=1)
                _view(mem, a["dst"]).copy_(torch.from_numpy(r.astype(np.int64)).reshape(a["dst"].shape))
            else:
                raise NotImplementedError(f"emulator: step kind '{k}'")
        by_buf = {}
        for oi, (bid, shape, dtype) in enumerate(plan.outputs):
            if bid not in by_buf:
                n = int(np.prod(shape)) if len(shape) else 1
                by_buf[bid] = mem[bid][:n].reshape(shape)
            outs[oi] = by_buf[bid]
        return outs


class EmulatorExecutor:
    """Drop-in for the HIP executor in CPU tests of the host logic."""

    name = "emulator"

    def __init__(self):
        self.torch_device = torch.device("cpu")
        self.rng_state = [0, 0]

    def seed(self, value: int) -> None:
        self.rng_state[:] = [int(value) & 0xFFFFFFFFFFFFFFFF, 0]

    def bind(self, plan: Plan) -> EmulatedPlan:
        return EmulatedPlan(plan, self.rng_state)

    def current_stream(self) -> int:
        return 0

    def synchronize(self) -> None:
        pass

    def check_status(self) -> None:
        pass
