#!/usr/bin/env python3
"""Generate straight-line 64-point DCT-II / DCT-III device code (dct64_gen.h).

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
log N.  Rotations are three lifting steps (three fused multiply-adds):
  x1 = x + p y, y1 = y - s x1, x2 = x1 + p y1,  p = tan(theta / 2).

Scaling.  The generated transforms are sqrt(32) TIMES the orthonormal ones:
only the DC term carries a multiplier (1/sqrt 2), the common factor sqrt(2/64)
is left out.  Two passes therefore give 32 times the orthonormal 2-D transform
and the kernels finish with an exact multiplication by 2^-5, on the selected
values only (encode) or folded into the scalar clip factor (decode).

The inverse transform is the transposed flow graph run backwards.

Functions written: dct64_fwd_head (the 32 input butterflies, from a separate
input array),
dct64_fwd_tail, dct64_fwd (both), dct64_inv, and dct64_inv_hooked (dct64_inv
with call-outs to a caller-supplied functor between its instructions); and, under TPLR_DCT_MATRIX_CORES, the
pieces of a measurement variant that computes the odd half of the forward transform (a 32-point DCT-IV, 47 % of
the operations) as a dense product on the matrix cores: dct64_fwd_even and the matrix kDct4Lane.  Run as a build step
(`python gen_dct64.py`); `--check` only verifies and prints op counts.
"""
from __future__ import annotations

import math
import os
import sys

import numpy as np

N = 64
GAIN = math.sqrt(N / 2.0)  # generated transform = GAIN * orthonormal transform


# --------------------------------------------------------------------------
# exact linear op list
#   ("bfly", i, j)        (s_i, s_j) <- (s_i + s_j, s_i - s_j)
#   ("rot", i, j, c, s)   (s_i, s_j) <- (c s_i + s s_j, -s s_i + c s_j)
#   ("mul", i, a)         s_i <- a s_i          (a = -1: sign flip, free)
# --------------------------------------------------------------------------
def build_forward():
    ops = []

    def c2(slots, dc):
        n = len(slots)
        if n == 1:
            if dc:
                ops.append(("mul", slots[0], 1.0 / math.sqrt(2.0)))
            return list(slots)
        h = n // 2
        for t in range(h):
            ops.append(("bfly", slots[t], slots[n - 1 - t]))
        even = c2([slots[t] for t in range(h)], dc)
        odd = c4([slots[n - 1 - t] for t in range(h)])
        out = [None] * n
        for m in range(h):
            out[2 * m] = even[m]
            out[2 * m + 1] = odd[m]
        return out

    def c4(slots):
        m = len(slots)
        if m == 1:
            ops.append(("mul", slots[0], math.cos(math.pi / 4)))
            return list(slots)
        half = m // 2
        for t in range(half):
            th = math.pi * (2 * t + 1) / (4 * m)
            ops.append(("rot", slots[t], slots[m - 1 - t], math.cos(th), math.sin(th)))
            if t & 1:
                ops.append(("mul", slots[m - 1 - t], -1.0))
        p = c2([slots[t] for t in range(half)], False)
        q = c2([slots[m - 1 - t] for t in range(half)], False)
        out = [None] * m
        out[0] = p[0]
        ops.append(("mul", q[0], -1.0))
        out[m - 1] = q[0]
        for j in range(1, half):
            ops.append(("bfly", p[j], q[half - j]))
            out[2 * j] = p[j]
            out[2 * j - 1] = q[half - j]
        return out

    # top level by hand so that the op list splits into head | even half | odd half
    h = N // 2
    slots = list(range(N))
    for t in range(h):
        ops.append(("bfly", slots[t], slots[N - 1 - t]))
    n_head = len(ops)
    even = c2([slots[t] for t in range(h)], True)
    n_even_end = len(ops)
    odd = c4([slots[N - 1 - t] for t in range(h)])
    out_slots = [None] * N
    for m in range(h):
        out_slots[2 * m] = even[m]
        out_slots[2 * m + 1] = odd[m]
    build_forward.split = (n_head, n_even_end)
    return ops, out_slots


def transpose_ops(ops):
    out = []
    for op in reversed(ops):
        if op[0] == "rot":
            _, i, j, c, s = op
            out.append(("rot", i, j, c, -s))
        else:
            out.append(op)  # butterflies and diagonal factors are symmetric
    return out


def run_ops(ops, x, dtype=np.float64, lifting=False):
    """Apply the op list to a slot-major state (one column per probe vector)."""
    x = x.astype(dtype).copy()
    f = dtype
    for op in ops:
        if op[0] == "mul":
            x[op[1]] = x[op[1]] * f(op[2])
        elif op[0] == "bfly":
            _, i, j = op
            a, b = x[i].copy(), x[j].copy()
            x[i], x[j] = a + b, a - b
        else:
            _, i, j, c, s = op
            a, b = x[i].copy(), x[j].copy()
            if lifting:
                p = f((1.0 - c) / s)
                a1 = a + p * b
                b1 = b - f(s) * a1
                x[i], x[j] = a1 + p * b1, b1
            else:
                x[i], x[j] = f(c) * a + f(s) * b, f(c) * b - f(s) * a
    return x


def as_matrix(ops, in_slots, out_slots, **kw):
    x = np.zeros((N, N))
    for n, s in enumerate(in_slots):
        x[s, n] = 1.0
    x = run_ops(ops, x, **kw)
    return np.stack([x[s] for s in out_slots])


def dense_dct():
    i = np.arange(N)[:, None]
    k = np.arange(N)[None, :]
    f = np.cos(np.pi * (2 * i + 1) * k / (2 * N)) * math.sqrt(2.0 / N)
    f[:, 0] = math.sqrt(1.0 / N)
    return f  # f[i, k]; forward = f.T @ x


# --------------------------------------------------------------------------
# emission with lazy sign tracking
# --------------------------------------------------------------------------
def lit(v):
    return np.format_float_scientific(np.float32(v), unique=True, trim="0") + "f"


class Emitter:
    def __init__(self, prefix, decl="const float"):
        self.lines, self.nops, self.n, self.prefix, self.decl = [], 0, 0, prefix, decl

    def emit(self, expr):
        self.n += 1
        name = f"{self.prefix}{self.n}"
        self.lines.append(f"    {self.decl} {name} = {expr};")
        self.nops += 1
        return name


N_HOOKS = 48  # call-outs spread evenly through dct64_inv_hooked


def emit_ops(em, ops, var, sign, hooks=0):
    hook_at = {(h * len(ops)) // hooks: h for h in range(hooks)} if hooks else {}
    for n_op, op in enumerate(ops):
        if n_op in hook_at:
            # Arithmetic has no ordering of its own against the memory operations of the hook, and
            # the compiler would slide all of it to one side.  Passing the 64 live values through an
            # empty asm statement (no instruction) before the hook keeps them where they are written.
            live = sorted(set(var.values()))
            for i in range(0, len(live), 16):
                em.lines.append("    asm volatile(\"\" : " + ", ".join(f'"+v"({x})' for x in live[i:i + 16]) + ");")
            em.lines.append(f"    hook(DctHook<{hook_at[n_op]}>{{}});")
        if op[0] == "mul":
            _, i, a = op
            a *= sign[i]
            if abs(abs(a) - 1.0) < 1e-15:
                sign[i] = math.copysign(1.0, a)
            else:
                var[i], sign[i] = em.emit(f"{var[i]} * {lit(a)}"), 1.0
        elif op[0] == "bfly":
            _, i, j = op
            xi, xj, si, sj = var[i], var[j], sign[i], sign[j]
            if si > 0 and sj > 0:
                var[i], sign[i] = em.emit(f"{xi} + {xj}"), 1.0
                var[j], sign[j] = em.emit(f"{xi} - {xj}"), 1.0
            elif si > 0:
                var[i], sign[i] = em.emit(f"{xi} - {xj}"), 1.0
                var[j], sign[j] = em.emit(f"{xi} + {xj}"), 1.0
            elif sj > 0:
                var[i], sign[i] = em.emit(f"{xj} - {xi}"), 1.0
                var[j], sign[j] = em.emit(f"{xi} + {xj}"), -1.0
            else:
                var[i], sign[i] = em.emit(f"{xi} + {xj}"), -1.0
                var[j], sign[j] = em.emit(f"{xj} - {xi}"), 1.0
        else:
            _, i, j, c, s = op
            s = s * sign[i] * sign[j]  # R diag(si, sj) = diag(si, sj) R(s -> s si sj)
            p = (1.0 - c) / s
            x1 = em.emit(f"__builtin_fmaf({var[j]}, {lit(p)}, {var[i]})")
            y1 = em.emit(f"__builtin_fmaf({x1}, {lit(-s)}, {var[j]})")
            x2 = em.emit(f"__builtin_fmaf({y1}, {lit(p)}, {x1})")
            var[i], var[j] = x2, y1


def finish(em, var, sign, out_slots, dst="v"):
    tail = []
    negs = 0
    for k, s in enumerate(out_slots):
        if sign[s] < 0:
            tail.append(f"    {dst}[{k}] = -{var[s]};")
            negs += 1
        else:
            tail.append(f"    {dst}[{k}] = {var[s]};")
    return "\n".join(em.lines + tail), negs


def emit_function(name, ops, in_slots, out_slots, hooks=0):
    em = Emitter("t", "float" if hooks else "const float")
    var = {s: f"v[{n}]" for n, s in enumerate(in_slots)}
    sign = {s: 1.0 for s in in_slots}
    emit_ops(em, ops, var, sign, hooks)
    body, negs = finish(em, var, sign, out_slots)
    if hooks:
        head = (f"template <typename Hook>\n__device__ __forceinline__ void {name}(float (&v)[64], Hook&& hook) {{")
    else:
        head = f"__device__ __forceinline__ void {name}(float (&v)[64]) {{"
    return f"{head}\n{body}\n}}\n", em.nops, negs


def emit_split_forward(ops, out_slots, n_head):
    """head: in[] -> v[] through the first n_head ops (slot order kept); tail: the rest, in place."""
    em = Emitter("h")
    var = {s: f"in[{s}]" for s in range(N)}
    sign = {s: 1.0 for s in range(N)}
    emit_ops(em, ops[:n_head], var, sign)
    assert all(sg > 0 for sg in sign.values())
    body, _ = finish(em, var, sign, list(range(N)))
    head = ("__device__ __forceinline__ void dct64_fwd_head(const float (&in)[64], float (&v)[64]) {\n"
            f"{body}\n}}\n")
    em2 = Emitter("t")
    var = {s: f"v[{s}]" for s in range(N)}
    sign = {s: 1.0 for s in range(N)}
    emit_ops(em2, ops[n_head:], var, sign)
    body, negs = finish(em2, var, sign, out_slots)
    tail = f"__device__ __forceinline__ void dct64_fwd_tail(float (&v)[64]) {{\n{body}\n}}\n"
    return head, tail, em.nops, em2.nops, negs


def emit_matrix_variant(fwd, out_slots, n_head, n_even_end):
    """Pieces for the measurement variant whose odd half (the 32-point DCT-IV of the differences) is a dense
    32x32 product on the matrix cores: the even half of the forward transform and the DCT-IV matrix."""
    h = N // 2
    # forward even half: slots 0..31 hold the sums after the head; even outputs are out[2m]
    em = Emitter("t")
    var = {s_: f"v[{s_}]" for s_ in range(h)}
    sign = {s_: 1.0 for s_ in range(h)}
    emit_ops(em, fwd[n_head:n_even_end], var, sign)
    lines = list(em.lines)
    for m in range(h):
        s_ = out_slots[2 * m]
        lines.append(f"    out[{2 * m}] = {'-' if sign[s_] < 0 else ''}{var[s_]};")
    f_even = ("__device__ __forceinline__ void dct64_fwd_even(const float (&v)[64], float (&out)[64]) {\n"
              + "\n".join(lines) + "\n}\n")
    # DCT-IV matrix C4[m][n] = cos(pi (2n+1)(2m+1) / (4*32)), symmetric.  Stored the way the
    # 32x32x2 matrix instruction wants its A operand: for K-step s, lane l supplies
    # A[i = l % 32][k = l / 32] = C4[l % 32][2 s + l / 32]; one row of 16 floats per lane.
    rows = []
    for l in range(64):
        m = l % 32
        rows.append("    {" + ", ".join(
            lit(math.cos(math.pi * (2 * (2 * s_ + l // 32) + 1) * (2 * m + 1) / (4 * h))) for s_ in range(16)) + "},")
    table = ("// 32-point DCT-IV C4[m][n] = cos(pi (2n+1)(2m+1) / 128), the odd half of the transform,\n"
             "// as A operands of v_mfma_f32_32x32x2_f32: kDct4Lane[l][s] = C4[l % 32][2 s + l / 32]\n"
             "__device__ const float kDct4Lane[64][16] = {\n" + "\n".join(rows) + "\n};\n")
    return f_even, table, em.nops


def main():
    check_only = "--check" in sys.argv
    fwd, out_slots = build_forward()
    inv = transpose_ops(fwd)
    ident = list(range(N))
    n_head, n_even_end = build_forward.split
    assert n_head == N // 2 and all(op[0] == "bfly" for op in fwd[:n_head])

    f = dense_dct()
    for lifting in (False, True):
        m_fwd = as_matrix(fwd, ident, out_slots, lifting=lifting)  # [k, n]
        m_inv = as_matrix(inv, out_slots, ident, lifting=lifting)
        err_f = np.abs(m_fwd - GAIN * f.T).max()
        err_i = np.abs(m_inv - GAIN * f).max()
        assert err_f < 1e-13 and err_i < 1e-13, (lifting, err_f, err_i)

    # float32 behaviour on heavy-tailed data, forward and round trip
    rng = np.random.default_rng(0)
    x = rng.standard_t(3, size=(N, 4096)) * 1e-3
    st = np.zeros((N, 4096))
    st[ident] = x
    y32 = run_ops(fwd, st, np.float32, lifting=True)
    y = np.stack([y32[s] for s in out_slots]).astype(np.float64) / GAIN
    y64 = f.T @ x
    rel = np.abs(y - y64).max() / np.abs(y64).max()
    st2 = np.zeros((N, 4096), np.float32)
    for k, s in enumerate(out_slots):
        st2[s] = y32[s]
    back = run_ops(inv, st2, np.float32, lifting=True)[ident].astype(np.float64) / (GAIN * GAIN)
    rel_rt = np.abs(back - x).max() / np.abs(x).max()

    # matrix-core variant of the forward transform: head butterflies, even half by the op list, odd half as
    # a dense 32-point DCT-IV of d[n] = slot[63 - n]
    h = N // 2
    c4 = np.cos(np.pi * np.outer(2 * np.arange(h) + 1, 2 * np.arange(h) + 1) / (4 * h))
    st = np.zeros((N, 4096))
    st[ident] = x
    st = run_ops(fwd[:n_even_end], st, np.float64, lifting=True)
    y_mm = np.zeros((N, 4096))
    y_mm[0::2] = st[[out_slots[2 * m] for m in range(h)]]
    y_mm[1::2] = c4 @ st[[N - 1 - n for n in range(h)]]
    err_mm_f = np.abs(y_mm / GAIN - y64).max() / np.abs(y64).max()
    assert err_mm_f < 1e-12, err_mm_f

    head, tail, n_h, n_t, neg_f = emit_split_forward(fwd, out_slots, n_head)
    t_inv, n_inv, neg_i = emit_function("dct64_inv", inv, out_slots, ident)
    t_inv_hooked, _, _ = emit_function("dct64_inv_hooked", inv, out_slots, ident, hooks=N_HOOKS)
    f_even, table, n_fe = emit_matrix_variant(fwd, out_slots, n_head, n_even_end)
    print(f"dct64_fwd: {n_h} + {n_t} ops (+{neg_f} negations), dct64_inv: {n_inv} ops (+{neg_i} negations)")
    print(f"matrix-core variant of dct64_fwd: 64 butterflies, even half {n_fe} ops, odd half = 32x32 DCT-IV")
    print(f"fp64 matrix error fwd {err_f:.2e} inv {err_i:.2e}; fp32 forward err / max|y| = {rel:.2e}, "
          f"round trip err / max|x| = {rel_rt:.2e}")
    if check_only:
        return
    here = os.path.dirname(os.path.abspath(__file__))
    with open(os.path.join(here, "dct64_gen.h"), "w") as fh:
        fh.write(
            "// Generated by gen_dct64.py - do not edit.\n"
            "// 64-point DCT-II (dct64_fwd = dct64_fwd_head + dct64_fwd_tail) and DCT-III (dct64_inv) as\n"
            "// straight-line butterfly / lifting-rotation code on the 64 registers of one lane.\n"
            "// Both are sqrt(32) times the orthonormal transform: two passes give 32x, and the caller\n"
            "// finishes with an exact multiplication by kDctPow2Scale.\n"
            f"// {n_h + n_t} / {n_inv} floating-point instructions per transform.\n"
            "#pragma once\n\n"
            "constexpr float kDctPow2Scale = 0.03125f;  // 2^-5\n\n"
        )
        fh.write(head + "\n" + tail + "\n")
        fh.write("__device__ __forceinline__ void dct64_fwd(float (&v)[64]) {\n"
                 "    float t[64];\n    dct64_fwd_head(v, t);\n    dct64_fwd_tail(t);\n"
                 "#pragma unroll\n    for (int i = 0; i < 64; ++i) v[i] = t[i];\n}\n\n")
        fh.write(t_inv)
        fh.write("\n// The same instructions with call-outs: hook(DctHook<h>{}) for h = 0 .. kDctHooks - 1, evenly spread,\n"
                 "// the first before any arithmetic.  A caller threads latency-bound work (LDS round trips, loads)\n"
                 "// through the transform that way; the results are bitwise those of dct64_inv.\n"
                 "template <int I>\nstruct DctHook {\n    static constexpr int value = I;\n};\n"
                 f"constexpr int kDctHooks = {N_HOOKS};\n\n")
        fh.write(t_inv_hooked)
        fh.write("\n// Measurement variant (TPLR_DCT_MATRIX_CORES): the odd half of dct64_fwd as a dense product on the\n"
                 "// matrix cores; see dct64_fwd_matrix in tplr_device.h.\n#if TPLR_DCT_MATRIX_CORES\n")
        fh.write(table + "\n" + f_even + "#endif\n")


if __name__ == "__main__":
    main()
