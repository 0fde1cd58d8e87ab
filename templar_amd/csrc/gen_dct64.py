#!/usr/bin/env python3
"""Generate straight-line 64-point orthonormal DCT-II / DCT-III device code.

The codec transforms every 64x64 chunk with F^T X F where
F[i,k] = c_k cos(pi (2i+1) k / 128), c_0 = sqrt(1/64), c_k = sqrt(2/64)
(reference: src/tplr/compress.py:710-741 builds the same matrix through an FFT,
src/tplr/compress.py:186-203 applies it).  A dense 64x64x64 contraction per
pass is compute bound on gfx950, so the kernels use a factorised transform in
which one lane owns one 64-vector in registers:

  C2_N(x)[2m]   = C2_{N/2}(u)[m],  u[n] = x[n] + x[N-1-n]
  C2_N(x)[2m+1] = C4_{N/2}(v)[m],  v[n] = x[n] - x[N-1-n]
  C4_M(v): rotate the pair (v[n], v[M-1-n]) by theta_n = pi (2n+1) / (4M)
           p[n] = v[n] cos + v[M-1-n] sin,  q[n] = (-1)^n (-v[n] sin + v[M-1-n] cos)
           P = C2_{M/2}(p), Q = C2_{M/2}(q)
           C4[0] = P[0], C4[M-1] = -Q[0],
           C4[2j] = P[j] + Q[M/2-j], C4[2j-1] = P[j] - Q[M/2-j]   (j = 1..M/2-1)

Every factor is a butterfly or a plane rotation, so rounding error grows like
log N.  The orthonormal scale factors are folded into the rotation constants
(one explicit multiply is left, on the DC term).  The inverse transform is the
transposed flow graph run backwards.

Output: dct64_gen.h next to this file.  Run as a build step
(`python gen_dct64.py`); `--check` only verifies and prints op counts.
"""
from __future__ import annotations

import math
import os
import sys

import numpy as np

N = 64


# --------------------------------------------------------------------------
# exact linear op list:  ("lin2", i, j, a, b, c, d)  (s_i, s_j) <- (a s_i + b s_j, c s_i + d s_j)
#                        ("mul", i, a)               s_i <- a s_i
# --------------------------------------------------------------------------
def build_forward():
    """Orthonormal DCT-II: the scale sigma = sqrt(2/N) rides down the recursion and is
    absorbed by the first rotation on every path; only the DC path has none, and gets
    one multiply by sqrt(1/N)."""
    ops = []
    sigma = math.sqrt(2.0 / N)

    def bfly(i, j):
        ops.append(("lin2", i, j, 1.0, 1.0, 1.0, -1.0))

    def c2(slots, scale, dc):
        n = len(slots)
        if n == 1:
            s = scale / math.sqrt(2.0) if dc else scale
            if s != 1.0:
                ops.append(("mul", slots[0], s))
            return list(slots)
        h = n // 2
        for t in range(h):
            bfly(slots[t], slots[n - 1 - t])
        even = c2([slots[t] for t in range(h)], scale, dc)
        odd = c4([slots[n - 1 - t] for t in range(h)], scale)
        out = [None] * n
        for m in range(h):
            out[2 * m] = even[m]
            out[2 * m + 1] = odd[m]
        return out

    def c4(slots, scale):
        m = len(slots)
        if m == 1:
            ops.append(("mul", slots[0], math.cos(math.pi / 4) * scale))
            return list(slots)
        half = m // 2
        for t in range(half):
            th = math.pi * (2 * t + 1) / (4 * m)
            c, s = math.cos(th) * scale, math.sin(th) * scale
            sg = -1.0 if (t & 1) else 1.0
            ops.append(("lin2", slots[t], slots[m - 1 - t], c, s, -sg * s, sg * c))
        p = c2([slots[t] for t in range(half)], 1.0, False)
        q = c2([slots[m - 1 - t] for t in range(half)], 1.0, False)
        out = [None] * m
        out[0] = p[0]
        ops.append(("mul", q[0], -1.0))
        out[m - 1] = q[0]
        for j in range(1, half):
            bfly(p[j], q[half - j])
            out[2 * j] = p[j]
            out[2 * j - 1] = q[half - j]
        return out

    out_slots = c2(list(range(N)), sigma, True)
    return ops, out_slots


def is_pm1(x):
    return abs(abs(x) - 1.0) < 1e-15


def transpose_ops(ops):
    out = []
    for op in reversed(ops):
        if op[0] == "mul":
            out.append(op)
        else:
            _, i, j, a, b, c, d = op
            out.append(("lin2", i, j, a, c, b, d))
    return out


def as_matrix(ops, in_slots, out_slots, dtype=np.float64):
    """Column k of the result = transform of unit vector k (inputs in logical order)."""
    x = np.zeros((N, N), dtype=dtype)  # slot-major state, one column per probe
    for n, s in enumerate(in_slots):
        x[s, n] = 1.0
    x = run_ops(ops, x, dtype)
    return np.stack([x[s] for s in out_slots])


def run_ops(ops, x, dtype=np.float64):
    x = x.astype(dtype).copy()
    for op in ops:
        if op[0] == "mul":
            _, i, a = op
            x[i] = (x[i] * dtype(a)).astype(dtype)
        else:
            _, i, j, a, b, c, d = op
            xi, xj = x[i].copy(), x[j].copy()
            x[i] = (dtype(a) * xi + dtype(b) * xj).astype(dtype)
            x[j] = (dtype(c) * xi + dtype(d) * xj).astype(dtype)
    return x


def dense_dct():
    i = np.arange(N)[:, None]
    k = np.arange(N)[None, :]
    f = np.cos(np.pi * (2 * i + 1) * k / (2 * N)) * math.sqrt(2.0 / N)
    f[:, 0] = math.sqrt(1.0 / N)
    return f  # f[i, k]; forward = f.T @ x


# --------------------------------------------------------------------------
# emission with lazy sign tracking and FMA fusion
# --------------------------------------------------------------------------
class Emitter:
    def __init__(self):
        self.lines = []
        self.nops = 0
        self.ntmp = 0

    def new(self):
        self.ntmp += 1
        return f"t{self.ntmp}"

    @staticmethod
    def lit(v):
        s = repr(float(np.float32(v)))
        if "e" not in s and "." not in s:
            s += ".0"
        # shortest repr of the float32 value, as a float literal
        s = np.format_float_scientific(np.float32(v), unique=True, trim="0")
        return s + "f"

    def emit(self, expr):
        name = self.new()
        self.lines.append(f"    const float {name} = {expr};")
        self.nops += 1
        return name


def emit_function(name, ops, in_slots, out_slots):
    """in_slots[n]: slot that input v[n] starts in; out_slots[k]: slot holding output k."""
    em = Emitter()
    var = {}
    sign = {}
    for n, s in enumerate(in_slots):
        var[s] = f"v[{n}]"
        sign[s] = 1.0
    for op in ops:
        if op[0] == "mul":
            _, i, a = op
            a = a * sign[i]
            if is_pm1(a):
                sign[i] = math.copysign(1.0, a)
                continue
            var[i] = em.emit(f"{var[i]} * {em.lit(a)}")
            sign[i] = 1.0
            continue
        _, i, j, a, b, c, d = op
        a, c = a * sign[i], c * sign[i]
        b, d = b * sign[j], d * sign[j]
        xi, xj = var[i], var[j]
        if all(is_pm1(v) for v in (a, b, c, d)):
            def row(p, q):
                # returns (expr, sign) for p*xi + q*xj with p,q in +-1
                if p > 0 and q > 0:
                    return f"{xi} + {xj}", 1.0
                if p > 0 and q < 0:
                    return f"{xi} - {xj}", 1.0
                if p < 0 and q > 0:
                    return f"{xj} - {xi}", 1.0
                return f"{xi} + {xj}", -1.0
            e1, s1 = row(a, b)
            e2, s2 = row(c, d)
            var[i], sign[i] = em.emit(e1), s1
            var[j], sign[j] = em.emit(e2), s2
        else:
            def row(p, q):
                # p*xi + q*xj with FMA; a +-1 coefficient saves the multiply
                if is_pm1(p):
                    base = xi if p > 0 else f"-{xi}"
                    return em.emit(f"__builtin_fmaf({xj}, {em.lit(q)}, {base})")
                if is_pm1(q):
                    base = xj if q > 0 else f"-{xj}"
                    return em.emit(f"__builtin_fmaf({xi}, {em.lit(p)}, {base})")
                t = em.emit(f"{xi} * {em.lit(p)}")
                return em.emit(f"__builtin_fmaf({xj}, {em.lit(q)}, {t})")
            n1 = row(a, b)
            n2 = row(c, d)
            var[i], sign[i] = n1, 1.0
            var[j], sign[j] = n2, 1.0
    tail = []
    negs = 0
    for k, s in enumerate(out_slots):
        if sign[s] < 0:
            tail.append(f"    v[{k}] = -{var[s]};")
            negs += 1
        else:
            tail.append(f"    v[{k}] = {var[s]};")
    body = "\n".join(em.lines + tail)
    text = (
        f"__device__ __forceinline__ void {name}(float (&v)[64]) {{\n{body}\n}}\n"
    )
    return text, em.nops, negs


def main():
    check_only = "--check" in sys.argv
    fwd, out_slots = build_forward()
    inv = transpose_ops(fwd)
    ident = list(range(N))

    f = dense_dct()
    m_fwd = as_matrix(fwd, ident, out_slots)  # [k, n]
    err_f = np.abs(m_fwd - f.T).max()
    m_inv = as_matrix(inv, out_slots, ident)  # inputs logical k live in out_slots[k]
    err_i = np.abs(m_inv - f).max()
    assert err_f < 1e-14 and err_i < 1e-14, (err_f, err_i)

    # float32 behaviour on heavy-tailed data
    rng = np.random.default_rng(0)
    x = (rng.standard_t(3, size=(N, 4096)) * 1e-3)
    st = np.zeros((N, 4096))
    st[ident] = x
    y32 = run_ops(fwd, st, np.float32)
    y32 = np.stack([y32[s] for s in out_slots]).astype(np.float64)
    y64 = f.T @ x
    rel = np.abs(y32 - y64).max() / np.abs(y64).max()

    t_fwd, n_fwd, neg_f = emit_function("dct64_fwd", fwd, ident, out_slots)
    t_inv, n_inv, neg_i = emit_function("dct64_inv", inv, out_slots, ident)
    print(f"dct64_fwd: {n_fwd} ops (+{neg_f} negations), dct64_inv: {n_inv} ops (+{neg_i} negations)")
    print(f"fp64 matrix error fwd {err_f:.2e} inv {err_i:.2e}; fp32 max err / max|y| = {rel:.2e}")
    if check_only:
        return
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "dct64_gen.h"), "w") as fh:
        fh.write(
            "// Generated by gen_dct64.py - do not edit.\n"
            "// 64-point orthonormal DCT-II (dct64_fwd) and its inverse, DCT-III (dct64_inv),\n"
            "// as straight-line butterfly/rotation code on 64 registers of one lane.\n"
            f"// {n_fwd} / {n_inv} floating-point instructions per transform.\n"
            "#pragma once\n\n"
        )
        fh.write(t_fwd)
        fh.write("\n")
        fh.write(t_inv)


if __name__ == "__main__":
    main()
