"""Writes tests/golden/kat.json: known-answer vectors for the hot-path operators.

The expected values are computed here from the ONNX-level DEFINITION of each
operator in exact rational arithmetic (fractions.Fraction) — direct convolution,
index permutation, windowed maximum — not by any code of this repository and
not by restating the reference's loops.  Inputs are small integers or dyadic
fractions, so every partial sum is exactly representable in fp32: any correct
implementation, whatever its summation order or accumulator width, must
reproduce the expected bits.  (The reference commits no expected values for
these operators; its only vector, Relu [-2,-0.5,0,1,3] -> [0,0,0,1,3] from
test/unit/cpuOperator.test.ts:15-18, is included as is.)

Run:  python tests/golden/make_golden.py
"""
import itertools
import json
import os
import random
import struct
from fractions import Fraction

HERE = os.path.dirname(os.path.abspath(__file__))


def f32(x):
    """Correctly rounded fp32 value of an exact rational (via double: exact for our sizes)."""
    return struct.unpack("<f", struct.pack("<f", float(x)))[0]


def rand_tensor(rng, shape, lo=-4, hi=4, denom=1):
    n = 1
    for s in shape:
        n *= s
    return [Fraction(rng.randint(lo * denom, hi * denom), denom) for _ in range(n)]


def strides_of(shape):
    st, acc = [], 1
    for s in reversed(shape):
        st.insert(0, acc)
        acc *= s
    return st


def at(data, shape, idx):
    st = strides_of(shape)
    return data[sum(i * s for i, s in zip(idx, st))]


def bcast_at(data, shape, out_idx):
    """numpy-style broadcast read of `data` (shape) at an index of the larger result."""
    pad = len(out_idx) - len(shape)
    idx = [0 if shape[d] == 1 else out_idx[pad + d] for d in range(len(shape))]
    return at(data, shape, idx) if shape else data[0]


def flt(values):
    return [float(v) for v in values]


def gemm_case(rng, m, n, k, trans_a, trans_b, alpha, beta, c_shape):
    a_shape = [k, m] if trans_a else [m, k]
    b_shape = [n, k] if trans_b else [k, n]
    A, B = rand_tensor(rng, a_shape), rand_tensor(rng, b_shape)
    C = rand_tensor(rng, c_shape) if c_shape is not None else None
    Y = []
    for i in range(m):
        for j in range(n):
            s = Fraction(0)
            for x in range(k):
                a = at(A, a_shape, [x, i] if trans_a else [i, x])
                b = at(B, b_shape, [j, x] if trans_b else [x, j])
                s += a * b
            y = Fraction(alpha) * s
            if C is not None:
                y += Fraction(beta) * bcast_at(C, c_shape, [i, j])
            Y.append(f32(y))
    return {"op": "Gemm", "A": flt(A), "A_shape": a_shape, "B": flt(B), "B_shape": b_shape,
            "C": flt(C) if C is not None else None, "C_shape": c_shape, "alpha": alpha, "beta": beta,
            "transA": trans_a, "transB": trans_b, "Y": Y, "Y_shape": [m, n]}


def matmul_case(rng, a_shape, b_shape):
    A, B = rand_tensor(rng, a_shape), rand_tensor(rng, b_shape)
    ea = [1] + a_shape if len(a_shape) == 1 else list(a_shape)
    eb = b_shape + [1] if len(b_shape) == 1 else list(b_shape)
    nd = max(len(ea), len(eb))
    ea = [1] * (nd - len(ea)) + ea
    eb = [1] * (nd - len(eb)) + eb
    batch = [max(x, y) for x, y in zip(ea[:-2], eb[:-2])]
    m, k, n = ea[-2], ea[-1], eb[-1]
    Y = []
    for bidx in itertools.product(*[range(b) for b in batch]):
        for i in range(m):
            for j in range(n):
                s = Fraction(0)
                for x in range(k):
                    ia = [0 if ea[d] == 1 else bidx[d] for d in range(nd - 2)] + [i, x]
                    ib = [0 if eb[d] == 1 else bidx[d] for d in range(nd - 2)] + [x, j]
                    s += at(A, ea, ia) * at(B, eb, ib)
                Y.append(f32(s))
    y_shape = batch + [m, n]
    if len(a_shape) == 1:
        del y_shape[-2]
    if len(b_shape) == 1:
        del y_shape[-1]
    return {"op": "MatMul", "A": flt(A), "A_shape": a_shape, "B": flt(B), "B_shape": b_shape,
            "Y": Y, "Y_shape": y_shape}


def conv_case(rng, n, c, h, w, cout, kh, kw, pads, strides, dilations, group, bias):
    x_shape, w_shape = [n, c, h, w], [cout, c // group, kh, kw]
    X, W = rand_tensor(rng, x_shape, -3, 3), rand_tensor(rng, w_shape, -2, 2)
    Bv = rand_tensor(rng, [cout]) if bias else None
    oh = (h + pads[0] + pads[2] - dilations[0] * (kh - 1) - 1) // strides[0] + 1
    ow = (w + pads[1] + pads[3] - dilations[1] * (kw - 1) - 1) // strides[1] + 1
    cg, og = c // group, cout // group
    Y = []
    for b in range(n):
        for co in range(cout):
            g = co // og
            for oy in range(oh):
                for ox in range(ow):
                    s = Fraction(0)
                    for ci in range(cg):
                        for ky in range(kh):
                            for kx in range(kw):
                                iy = oy * strides[0] - pads[0] + ky * dilations[0]
                                ix = ox * strides[1] - pads[1] + kx * dilations[1]
                                if 0 <= iy < h and 0 <= ix < w:
                                    s += at(X, x_shape, [b, g * cg + ci, iy, ix]) * at(W, w_shape, [co, ci, ky, kx])
                    if Bv is not None:
                        s += Bv[co]
                    Y.append(f32(s))
    return {"op": "Conv", "X": flt(X), "X_shape": x_shape, "W": flt(W), "W_shape": w_shape,
            "B": flt(Bv) if Bv is not None else None, "pads": pads, "strides": strides,
            "dilations": dilations, "group": group, "Y": Y, "Y_shape": [n, cout, oh, ow]}


def pool_geometry(size, k, strides, dilations, attrs):
    """Output size and begin-pads per the ONNX MaxPool specification."""
    auto_pad = attrs.get("auto_pad", "NOTSET")
    out, begin = [], []
    for a in range(2):
        eff = (k[a] - 1) * dilations[a] + 1
        if auto_pad == "NOTSET":
            pads = attrs.get("pads", [0, 0, 0, 0])
            num = size[a] + pads[a] + pads[a + 2] - eff
            o = (-(-num // strides[a]) if attrs.get("ceil_mode", 0) else num // strides[a]) + 1
            out.append(o)
            begin.append(pads[a])
        elif auto_pad == "VALID":
            out.append(-(-(size[a] - eff + 1) // strides[a]))
            begin.append(0)
        else:
            o = -(-size[a] // strides[a])
            total = max((o - 1) * strides[a] + eff - size[a], 0)
            out.append(o)
            begin.append(total // 2 if auto_pad == "SAME_UPPER" else total - total // 2)
    return out, begin


def maxpool_case(rng, n, c, h, w, k, strides, dilations, attrs):
    (oh, ow), pads = pool_geometry([h, w], k, strides, dilations, attrs)
    x_shape = [n, c, h, w]
    X = rand_tensor(rng, x_shape, -50, 50, 2)
    Y = []
    for b in range(n):
        for ch in range(c):
            for oy in range(oh):
                for ox in range(ow):
                    best = None
                    for ky in range(k[0]):
                        for kx in range(k[1]):
                            iy = oy * strides[0] - pads[0] + ky * dilations[0]
                            ix = ox * strides[1] - pads[1] + kx * dilations[1]
                            if 0 <= iy < h and 0 <= ix < w:
                                v = at(X, x_shape, [b, ch, iy, ix])
                                best = v if best is None or v > best else best
                    Y.append(float(best) if best is not None else float("-inf"))
    case = {"op": "MaxPool", "X": flt(X), "X_shape": x_shape, "kernel_shape": k, "Y": Y,
            "Y_shape": [n, c, oh, ow]}
    case.update(attrs)
    return case


def transpose_case(rng, shape, perm):
    X = rand_tensor(rng, shape, -100, 100)
    out_shape = [shape[p] for p in perm]
    Y = []
    for idx in itertools.product(*[range(s) for s in out_shape]):
        src = [0] * len(shape)
        for o, p in enumerate(perm):
            src[p] = idx[o]
        Y.append(float(at(X, shape, src)))
    return {"op": "Transpose", "X": flt(X), "X_shape": shape, "perm": perm, "Y": Y, "Y_shape": out_shape}


def binary_case(rng, op, l_shape, r_shape):
    L = rand_tensor(rng, l_shape, -8, 8, 4)
    R = rand_tensor(rng, r_shape, -8, 8, 4)
    if op == "Div":
        # power-of-two divisors keep every quotient exactly representable
        R = [(Fraction(2) ** rng.randint(-2, 2)) * (1 if r > 0 else -1) for r in R]
    nd = max(len(l_shape), len(r_shape))
    el = [1] * (nd - len(l_shape)) + l_shape
    er = [1] * (nd - len(r_shape)) + r_shape
    out_shape = [max(a, b) for a, b in zip(el, er)]
    fn = {"Add": lambda a, b: a + b, "Sub": lambda a, b: a - b, "Mul": lambda a, b: a * b,
          "Div": lambda a, b: a / b}[op]
    Y = []
    for idx in itertools.product(*[range(s) for s in out_shape]):
        l, r = bcast_at(L, l_shape, list(idx)), bcast_at(R, r_shape, list(idx))
        y = f32(fn(l, r))
        # rationals have no signed zero; IEEE gives a zero product/quotient the XOR of the signs
        # (the zero operands here are all +0)
        if y == 0 and op in ("Mul", "Div") and (l < 0) != (r < 0):
            y = -0.0
        Y.append(y)
    return {"op": op, "L": flt(L), "L_shape": l_shape, "R": flt(R), "R_shape": r_shape, "Y": Y,
            "Y_shape": out_shape}


def gap_case(rng, n, c, h, w):
    shape = [n, c, h, w]
    X = rand_tensor(rng, shape, -64, 64, 8)
    Y = []
    for b in range(n):
        for ch in range(c):
            s = sum(at(X, shape, [b, ch, y, x]) for y in range(h) for x in range(w))
            Y.append(f32(s / (h * w)))
    return {"op": "GlobalAveragePool", "X": flt(X), "X_shape": shape, "Y": Y, "Y_shape": [n, c, 1, 1]}


def portable(obj):
    """Strict JSON has no infinities: they are written as the strings "inf" / "-inf"."""
    if isinstance(obj, float) and obj in (float("inf"), float("-inf")):
        return "inf" if obj > 0 else "-inf"
    if isinstance(obj, list):
        return [portable(o) for o in obj]
    if isinstance(obj, dict):
        return {k: portable(v) for k, v in obj.items()}
    return obj


def main():
    rng = random.Random(20240607)
    cases = []
    for ta, tb in itertools.product((0, 1), (0, 1)):
        cases.append(gemm_case(rng, 7, 5, 3, ta, tb, 1.0, 1.0, [5]))
    cases.append(gemm_case(rng, 2, 4, 3, 0, 0, 1.0, 1.0, [4]))       # test/fixtures/generate_fixtures.py:67-73 shape
    cases.append(gemm_case(rng, 6, 9, 20, 0, 1, 0.5, 2.0, [6, 1]))
    cases.append(gemm_case(rng, 6, 9, 20, 1, 0, 2.0, 0.25, [6, 9]))
    cases.append(gemm_case(rng, 5, 3, 4, 0, 0, 1.0, 1.0, [1]))
    cases.append(gemm_case(rng, 5, 3, 4, 0, 0, 1.0, 1.0, []))
    cases.append(gemm_case(rng, 5, 3, 4, 0, 0, 0.0, 1.0, [1, 3]))      # alpha = 0 -> beta*C
    cases.append(gemm_case(rng, 5, 3, 4, 1, 1, -1.5, 0.0, [3]))        # beta = 0 == no C
    cases.append(gemm_case(rng, 33, 35, 19, 0, 1, 1.0, 1.0, None))
    cases.append(matmul_case(rng, [3, 4], [4, 5]))
    cases.append(matmul_case(rng, [2, 3, 4], [4, 5]))
    cases.append(matmul_case(rng, [1, 3, 16], [4, 16, 1]))            # test/model_test/make_models.py:620
    cases.append(matmul_case(rng, [2, 3, 4], [2, 4, 2]))
    cases.append(matmul_case(rng, [4], [4, 3]))
    cases.append(matmul_case(rng, [2, 3, 4], [4]))
    cases.append(matmul_case(rng, [5], [5]))
    cases.append(conv_case(rng, 1, 1, 3, 3, 1, 2, 2, [0, 0, 0, 0], [1, 1], [1, 1], 1, False))  # generate_fixtures.py:88-104 shape
    cases.append(conv_case(rng, 2, 3, 6, 7, 4, 3, 3, [1, 1, 1, 1], [1, 1], [1, 1], 1, True))
    cases.append(conv_case(rng, 1, 4, 7, 6, 6, 3, 3, [1, 0, 2, 1], [2, 2], [1, 1], 2, True))
    cases.append(conv_case(rng, 1, 2, 9, 9, 3, 3, 3, [2, 2, 2, 2], [1, 1], [2, 2], 1, False))
    cases.append(conv_case(rng, 2, 4, 5, 5, 4, 3, 3, [1, 1, 1, 1], [1, 1], [1, 1], 4, True))     # depthwise
    cases.append(conv_case(rng, 1, 3, 12, 11, 5, 7, 7, [3, 3, 3, 3], [2, 2], [1, 1], 1, True))  # stem-like
    cases.append(conv_case(rng, 2, 6, 4, 5, 3, 1, 1, [0, 0, 0, 0], [2, 2], [1, 1], 1, False))   # 1x1 stride 2
    cases.append(maxpool_case(rng, 2, 3, 10, 12, [3, 3], [2, 2], [1, 1], {"strides": [2, 2]}))   # make_models.py:650
    cases.append(maxpool_case(rng, 2, 3, 10, 12, [3, 3], [2, 2], [1, 1],
                              {"strides": [2, 2], "ceil_mode": 1}))                              # make_models.py:652
    cases.append(maxpool_case(rng, 1, 2, 9, 9, [3, 3], [2, 2], [1, 1],
                              {"strides": [2, 2], "pads": [1, 1, 1, 1]}))                        # ResNet stem form
    for auto_pad in ("SAME_UPPER", "SAME_LOWER", "VALID"):
        cases.append(maxpool_case(rng, 1, 1, 7, 8, [3, 3], [2, 3], [1, 1],
                                  {"strides": [2, 3], "auto_pad": auto_pad}))
    cases.append(maxpool_case(rng, 1, 1, 9, 9, [2, 2], [2, 2], [2, 2],
                              {"strides": [2, 2], "dilations": [2, 2], "pads": [1, 1, 1, 1]}))
    # a window that lies wholly in the padding -> -inf: in=4, pads 1+1, k=2, s=3, ceil
    cases.append(maxpool_case(rng, 1, 1, 4, 4, [2, 2], [3, 3], [1, 1],
                              {"strides": [3, 3], "pads": [1, 1, 1, 1], "ceil_mode": 1}))
    cases.append(transpose_case(rng, [3, 4, 5], [2, 0, 1]))                                      # make_models.py:712
    cases.append(transpose_case(rng, [3, 4], [1, 0]))
    cases.append(transpose_case(rng, [2, 3, 4, 5], [0, 2, 1, 3]))
    cases.append(transpose_case(rng, [2, 3, 2, 2, 3], [4, 0, 3, 1, 2]))
    for op in ("Add", "Sub", "Mul", "Div"):
        cases.append(binary_case(rng, op, [2, 3, 4, 6], [1, 3, 1, 6]))
        cases.append(binary_case(rng, op, [2, 3, 4, 6], []))
        cases.append(binary_case(rng, op, [4, 1], [3]))
    cases.append(gap_case(rng, 2, 3, 7, 7))
    cases.append(gap_case(rng, 1, 4, 4, 8))
    cases.append({"op": "Relu", "X": [-2.0, -0.5, 0.0, 1.0, 3.0], "X_shape": [5],
                  "Y": [0.0, 0.0, 0.0, 1.0, 3.0], "Y_shape": [5],
                  "source": "test/unit/cpuOperator.test.ts:15-18"})
    cases.append({"op": "Softmax", "X": [1.5] * 8 + [-3.0] * 8, "X_shape": [2, 8],
                  "Y": [0.125] * 16, "Y_shape": [2, 8]})
    cases.append({"op": "Softmax", "X": [0.0, float("-inf"), float("-inf"), float("-inf"), 7.0,
                                         float("-inf")], "X_shape": [2, 3],
                  "Y": [1.0, 0.0, 0.0, 0.0, 1.0, 0.0], "Y_shape": [2, 3]})
    # rows with mean 0 and variance 1, eps = 0: y = x*gamma + beta exactly
    cases.append({"op": "LayerNormalization", "X": [1.0, -1.0, 1.0, -1.0, -1.0, -1.0, 1.0, 1.0],
                  "X_shape": [2, 4], "gamma": [2.0, 0.5, 1.0, -1.0], "beta": [0.0, 1.0, -2.0, 0.25],
                  "epsilon": 0.0, "Y": [2.0, 0.5, -1.0, 1.25, -2.0, 0.5, -1.0, -0.75], "Y_shape": [2, 4]})
    with open(os.path.join(HERE, "kat.json"), "w") as f:
        json.dump({"cases": portable(cases)}, f, allow_nan=False)
    print("wrote", len(cases), "cases")


if __name__ == "__main__":
    main()
