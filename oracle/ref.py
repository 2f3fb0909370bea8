"""TEST INFRASTRUCTURE ONLY — numpy face of the CPU oracle (oracle/webdnn_cpu_ref.c).

Only tests/, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import this module; the product (``webdnn_amd``) never does.

Each function takes ONNX-level arguments (numpy arrays + attributes) like the
reference operator it restates, returns a new numpy array, and raises
``RefThrows`` where the reference operator throws.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")


class RefThrows(Exception):
    """The reference operator would throw for these arguments."""


def build():
    subprocess.run(["make", "-C", _HERE, "-s", "-B"], check=True)
    return _LIB_PATH


def _load():
    if not os.path.exists(_LIB_PATH):
        build()
    return ctypes.CDLL(_LIB_PATH)


_lib = _load()
_i64p = ctypes.POINTER(ctypes.c_int64)
_vp = ctypes.c_void_p


def set_threads(n):
    """OpenMP threads for the outer loops (results do not depend on it)."""
    _lib.ref_set_threads(int(n))


def _dims(shape):
    arr = (ctypes.c_int64 * max(len(shape), 1))(*[int(s) for s in shape])
    return arr, len(shape)


def _ints(values):
    values = list(values) if values is not None else []
    arr = (ctypes.c_int64 * max(len(values), 1))(*[int(v) for v in values])
    return arr, len(values)


def _f32(a):
    a = np.asarray(a, dtype=np.float32, order="C")
    return a


def _ptr(a):
    return a.ctypes.data_as(_vp) if a is not None else None


def _check(rc, what):
    if rc == -2:
        raise MemoryError(what)
    if rc < 0:
        raise RefThrows(what)
    return rc


def gemm(A, B, C=None, alpha=1.0, beta=1.0, transA=0, transB=0):
    A, B = _f32(A), _f32(B)
    C = _f32(C) if C is not None else None
    dA, nA = _dims(A.shape)
    dB, nB = _dims(B.shape)
    dC, nC = _dims(C.shape) if C is not None else _dims(())
    m, n = ctypes.c_int64(), ctypes.c_int64()
    # attributes are fp32 in the ONNX file, read back as JS doubles
    alpha = float(np.float32(alpha))
    beta = float(np.float32(beta))
    args = lambda y: (_ptr(A), dA, nA, _ptr(B), dB, nB, _ptr(C), dC, nC,
                      ctypes.c_double(alpha), ctypes.c_double(beta), int(transA), int(transB),
                      y, ctypes.byref(m), ctypes.byref(n))
    _check(_lib.ref_gemm(*args(None)), "Gemm: shape")
    Y = np.empty((m.value, n.value), dtype=np.float32)
    _check(_lib.ref_gemm(*args(_ptr(Y))), "Gemm")
    return Y


def matmul(A, B):
    A, B = _f32(A), _f32(B)
    dA, nA = _dims(A.shape)
    dB, nB = _dims(B.shape)
    out = (ctypes.c_int64 * 8)()
    nd = _check(_lib.ref_matmul(_ptr(A), dA, nA, _ptr(B), dB, nB, None, out), "MatMul: shape")
    Y = np.empty(tuple(out[i] for i in range(nd)), dtype=np.float32)
    _check(_lib.ref_matmul(_ptr(A), dA, nA, _ptr(B), dB, nB, _ptr(Y), out), "MatMul")
    return Y


def conv(X, W, B=None, dilations=None, group=1, kernel_shape=None, pads=None, strides=None):
    X, W = _f32(X), _f32(W)
    B = _f32(B) if B is not None else None
    dX, nX = _dims(X.shape)
    dW, _ = _dims(W.shape)
    dil, ndil = _ints(dilations)
    ks, nks = _ints(kernel_shape)
    pd, npd = _ints(pads)
    st, nst = _ints(strides)
    out = (ctypes.c_int64 * 4)()
    args = lambda y: (_ptr(X), dX, nX, _ptr(W), dW, _ptr(B), dil, ndil, ctypes.c_int64(group),
                      ks, nks, pd, npd, st, nst, y, out)
    _check(_lib.ref_conv(*args(None)), "Conv: shape")
    Y = np.empty(tuple(out[i] for i in range(4)), dtype=np.float32)
    _check(_lib.ref_conv(*args(_ptr(Y))), "Conv")
    return Y


_BIN = {"Add": 0, "Sub": 1, "Mul": 2, "Div": 3, "Pow": 4}


def binary(op, L, R):
    L, R = np.asarray(L, order="C"), np.asarray(R, order="C")
    if L.dtype != R.dtype:
        raise RefThrows("Binary: input dataTypes mismatch")
    if L.dtype == np.float32:
        dtype = 0
    elif L.dtype == np.int32:
        dtype = 1
    else:
        raise RefThrows("Binary: dataType not supported")
    dL, nL = _dims(L.shape)
    dR, nR = _dims(R.shape)
    out = (ctypes.c_int64 * 8)()
    nd = _check(_lib.ref_binary(_BIN[op], dtype, _ptr(L), dL, nL, _ptr(R), dR, nR, None, out),
                "Binary: broadcast")
    Y = np.empty(tuple(out[i] for i in range(nd)), dtype=L.dtype)
    _check(_lib.ref_binary(_BIN[op], dtype, _ptr(L), dL, nL, _ptr(R), dR, nR, _ptr(Y), out), "Binary")
    return Y


_UN = {"Relu": 0, "Sigmoid": 1, "Sqrt": 2, "Exp": 3, "Tanh": 4, "Abs": 5, "Neg": 6, "Reciprocal": 7}


def unary(op, X):
    X = np.asarray(X, order="C")
    if X.dtype == np.float32:
        dtype = 0
    elif X.dtype == np.int32:
        dtype = 1
    else:
        raise RefThrows("Unary: DataType not supported")
    Y = np.empty_like(X)
    _check(_lib.ref_unary(_UN[op], dtype, _ptr(X), _ptr(Y), ctypes.c_int64(X.size)), "Unary")
    return Y


def softmax(X, axis=-1):
    X = _f32(X)
    d, n = _dims(X.shape)
    Y = np.empty_like(X)
    _check(_lib.ref_softmax(_ptr(X), d, n, ctypes.c_int64(axis), _ptr(Y)), "Softmax")
    return Y


_AUTO_PAD = {"NOTSET": 0, "SAME_UPPER": 1, "SAME_LOWER": 2, "VALID": 3}


def maxpool(X, kernel_shape, auto_pad="NOTSET", ceil_mode=0, dilations=None, pads=None,
            strides=None, n_outputs=1, return_pads=False):
    X = _f32(X)
    if auto_pad not in _AUTO_PAD:
        raise RefThrows("Unknown auto_pad")
    dX, nX = _dims(X.shape)
    dil, ndil = _ints(dilations)
    ks, _ = _ints(kernel_shape)
    pd, npd = _ints(pads)
    st, nst = _ints(strides)
    out = (ctypes.c_int64 * 4)()
    pads_out = (ctypes.c_int64 * 4)()
    args = lambda y: (_ptr(X), dX, nX, _AUTO_PAD[auto_pad], int(ceil_mode), dil, ndil, ks, pd, npd,
                      st, nst, int(n_outputs), y, out, pads_out)
    _check(_lib.ref_maxpool(*args(None)), "MaxPool: shape")
    Y = np.empty(tuple(out[i] for i in range(4)), dtype=np.float32)
    _check(_lib.ref_maxpool(*args(_ptr(Y))), "MaxPool")
    if return_pads:
        return Y, [pads_out[i] for i in range(4)]
    return Y


def global_average_pool(X):
    X = _f32(X)
    d, n = _dims(X.shape)
    if n != 4:
        raise RefThrows("GlobalAveragePool other than 2D")
    Y = np.empty((X.shape[0], X.shape[1], 1, 1), dtype=np.float32)
    _check(_lib.ref_global_average_pool(_ptr(X), d, n, _ptr(Y)), "GlobalAveragePool")
    return Y


def transpose(X, perm=None):
    X = np.asarray(X, order="C")
    assert X.dtype.itemsize == 4
    d, n = _dims(X.shape)
    pm, npm = _ints(perm)
    out = (ctypes.c_int64 * 8)()
    _check(_lib.ref_transpose(None, d, n, pm, npm, None, out), "Transpose: shape")
    Y = np.empty(tuple(out[i] for i in range(n)), dtype=X.dtype)
    _check(_lib.ref_transpose(_ptr(X), d, n, pm, npm, _ptr(Y), out), "Transpose")
    return Y


def reduce_mean_last(X):
    """ReduceMean over the last axis, keepdims=1."""
    X = _f32(X)
    length = X.shape[-1]
    outer = X.size // length if length else 0
    Y = np.empty(X.shape[:-1] + (1,), dtype=np.float32)
    _check(_lib.ref_reduce_mean_trailing(_ptr(X), ctypes.c_int64(outer), ctypes.c_int64(length),
                                         _ptr(Y)), "ReduceMean")
    return Y


def reduce_mean(X, axes=(), keepdims=1):
    """ReduceMean over any set of axes (all axes when `axes` is empty): one pass per axis in
    ascending order, fp32 between the passes (reduce.ts:40-100, 114-131, 369-405)."""
    X = _f32(X)
    nd = X.ndim
    ax = sorted(a + nd if a < 0 else a for a in axes) if len(axes) else list(range(nd))
    shape, data, total = list(X.shape), np.ascontiguousarray(X).reshape(-1), 1
    for i, a in enumerate(ax):
        red = shape[a]
        total *= red
        outer = int(np.prod(shape[:a], dtype=np.int64))
        inner = int(np.prod(shape[a + 1:], dtype=np.int64))
        out = np.empty(outer * inner, dtype=np.float32)
        divisor = float(total) if i == len(ax) - 1 else 1.0
        _check(_lib.ref_reduce_axis(_ptr(data), ctypes.c_int64(outer), ctypes.c_int64(red), ctypes.c_int64(inner),
                                    ctypes.c_double(divisor), _ptr(out)), "ReduceMean")
        shape[a], data = 1, out
    final = shape if keepdims else [d for i, d in enumerate(shape) if i not in ax]
    return data.reshape(final)


def gather(data, indices, axis=0):
    data = np.asarray(data, order="C")
    indices = np.asarray(indices, dtype=np.int32, order="C")
    Y = np.empty((), dtype=data.dtype)
    _check(_lib.ref_gather(_ptr(data), data.ndim, _ptr(indices), indices.ndim,
                           ctypes.c_int64(axis), _ptr(Y)), "Gather")
    return Y


def layernorm_decomposed(X, gamma=None, beta=None, eps=1e-5):
    X = _f32(X)
    gamma = _f32(gamma) if gamma is not None else None
    beta = _f32(beta) if beta is not None else None
    length = X.shape[-1]
    outer = X.size // length if length else 0
    Y = np.empty_like(X)
    _check(_lib.ref_layernorm_decomposed(_ptr(X), ctypes.c_int64(outer), ctypes.c_int64(length),
                                         _ptr(gamma), _ptr(beta), ctypes.c_float(eps), _ptr(Y)),
           "LayerNormalization")
    return Y


def flatten(X, axis=1):
    """operators/base/flatten.ts:7-17 + cpu flatten.ts:11-20 (shares the buffer)."""
    if axis != 1:
        raise RefThrows("Flatten: only axis === 1 is supported")
    X = np.asarray(X)
    return X.reshape(X.shape[0], int(np.prod(X.shape[1:], dtype=np.int64)))


def reshape(X, shape, allowzero=0):
    """operators/base/reshape5.ts:16-75, written out (no numpy -1 inference)."""
    X = np.asarray(X)
    shape = [int(s) for s in np.asarray(shape).reshape(-1)]
    explicit, minus = 1, -1
    for i, s in enumerate(shape):
        if s > 0:
            explicit *= s
        elif s == 0 and not allowzero:
            explicit *= X.shape[i]
        elif s == -1:
            if minus >= 0:
                raise RefThrows("Reshape: multiple -1 dimensions")
            minus = i
        elif s < -1:
            raise RefThrows("Reshape: negative dimension")
    if minus >= 0 and explicit <= 0:
        raise RefThrows("Reshape: cannot infer -1")
    out = []
    for i, s in enumerate(shape):
        if s > 0 or (s == 0 and allowzero):
            out.append(s)
        elif s == 0:
            out.append(X.shape[i])
        else:
            out.append(X.size // explicit)
    return X.reshape(out)


# ---- layout glue: pure index arithmetic, restated in numpy/python ------------------

def squeeze(X, axes=()):
    """operators/base/squeeze.ts:8-22 (+ cpu squeeze.ts:12-37: shares the buffer)."""
    X = np.asarray(X)
    axes = [int(a) for a in axes]
    if not axes:
        shape = [s for s in X.shape if s != 1]
    else:
        nn = [a if a >= 0 else a + X.ndim for a in axes]
        shape = [s for i, s in enumerate(X.shape) if i not in nn]
    if int(np.prod(shape, dtype=np.int64)) != X.size:
        raise RefThrows("Squeeze: removed axis is not of extent 1")  # emptyTensor(dims, type, data) length check
    return X.reshape(shape)


def unsqueeze(X, axes):
    """operators/base/unsqueeze.ts:8-27 (+ cpu unsqueeze.ts: shares the buffer)."""
    X = np.asarray(X)
    axes = [int(a) for a in axes]
    nd = X.ndim + len(axes)
    nn = [a if a >= 0 else a + nd for a in axes]
    shape, src = [], 0
    for d in range(nd):
        if d in nn:
            shape.append(1)
        else:
            if src >= X.ndim:
                raise RefThrows("Unsqueeze: axes out of range")
            shape.append(X.shape[src])
            src += 1
    if src != X.ndim:
        raise RefThrows("Unsqueeze: duplicate axes")
    return X.reshape(shape)


def concat(inputs, axis=0):
    """cpu concat.ts:21-84: the flat-index loops, vectorised over (c, outer, inner)."""
    inputs = [np.asarray(t, order="C") for t in inputs]
    first = inputs[0]
    ax = axis if axis >= 0 else first.ndim + axis
    if ax < 0 or ax >= first.ndim:
        raise RefThrows("Concat: axis %d out of range" % ax)
    out_shape = list(first.shape)
    out_shape[ax] = sum(t.shape[ax] for t in inputs)
    outer_len = int(np.prod(first.shape[:ax], dtype=np.int64))
    inner_len = int(np.prod(first.shape[ax + 1:], dtype=np.int64))

    def strides(shape):
        s, acc = [], 1
        for d in reversed(shape):
            s.insert(0, acc)
            acc *= d
        return s

    out = np.zeros(int(np.prod(out_shape, dtype=np.int64)), dtype=first.dtype)
    so = strides(out_shape)
    out_outer, out_cat = so[max(ax - 1, 0)], so[ax]
    offset = 0
    for t in inputs:
        st = strides(t.shape)
        dim, outer_s, cat_s = t.shape[ax], st[max(ax - 1, 0)], st[ax]
        c, o, i = np.meshgrid(np.arange(dim), np.arange(outer_len), np.arange(inner_len),
                              indexing="ij")
        out[((c + offset) * out_cat + o * out_outer + i).reshape(-1)] = \
            t.reshape(-1)[(c * cat_s + o * outer_s + i).reshape(-1)]
        offset += dim
    return out.reshape(out_shape)


def split(X, n_outputs, axis=0, split=()):
    """operators/base/split.ts:10-70 + cpu split.ts:12-45."""
    X = np.asarray(X, order="C")
    ax = axis if axis >= 0 else axis + X.ndim
    if ax < 0 or ax >= X.ndim:
        raise RefThrows("Split: axis %d out of range" % ax)
    axis_len = X.shape[ax]
    parts = [int(s) for s in split] if len(split) else [axis_len // n_outputs] * n_outputs
    outer_len = int(np.prod(X.shape[:ax], dtype=np.int64))
    inner_len = int(np.prod(X.shape[ax + 1:], dtype=np.int64))
    in_cat = inner_len
    # input.strides[max(axis-1, 0)]
    st, acc = [], 1
    for d in reversed(X.shape):
        st.insert(0, acc)
        acc *= d
    in_outer = st[max(ax - 1, 0)]
    flat = X.reshape(-1)
    outs, offset = [], 0
    for n in range(n_outputs):
        dim = parts[n]
        out_shape = list(X.shape)
        out_shape[ax] = dim
        outer_s = int(np.prod(out_shape[max(ax - 1, 0) + 1:], dtype=np.int64))
        split_s = int(np.prod(out_shape[ax + 1:], dtype=np.int64))
        ot = np.zeros(int(np.prod(out_shape, dtype=np.int64)), dtype=X.dtype)
        c, o, i = np.meshgrid(np.arange(dim), np.arange(outer_len), np.arange(inner_len),
                              indexing="ij")
        ot[(c * split_s + o * outer_s + i).reshape(-1)] = \
            flat[((c + offset) * in_cat + o * in_outer + i).reshape(-1)]
        outs.append(ot.reshape(out_shape))
        offset += dim
    return outs


def slice_(data, starts, ends, axes=None, steps=None):
    """cpu slice.ts:12-94 (Slice, opset >= 10), including its clamping rules:
    start is clamped to [0, size-1] and stop to [-1, size] whatever the sign of the step."""
    data = np.asarray(data, order="C")
    if data.ndim > 6:
        raise RefThrows("Slice: input dimension %d > 6 is not yet supported" % data.ndim)
    starts = [int(v) for v in starts]
    ends = [int(v) for v in ends]
    if axes is not None:
        axes = [int(a) + data.ndim if int(a) < 0 else int(a) for a in axes]
    else:
        axes = list(range(data.ndim))
    steps = [int(v) for v in steps] if steps is not None else [1] * len(axes)
    ranges = [[0, d, 1, d] for d in data.shape]
    for i, a in enumerate(axes):
        ranges[a] = [starts[i], ends[i], steps[i], data.shape[a]]
    index = []
    for start, stop, step, size in ranges:
        if start < 0:
            start += size
        start = max(min(start, size - 1), 0)
        if stop < 0:
            stop += size
        stop = max(min(stop, size), -1)
        dst = max(int(np.ceil((stop - start) / step)), 0)
        index.append(start + step * np.arange(dst))
    out_shape = [len(ix) for ix in index]
    if data.ndim == 0:
        return data.copy()
    return data[np.ix_(*index)].reshape(out_shape)


def js_to_int32(values):
    """ECMAScript ToInt32 of each element (what TypedArray.prototype.set does for Int32Array)."""
    v = np.asarray(values, dtype=np.float64)
    finite = np.isfinite(v)
    t = np.trunc(np.where(finite, v, 0.0))
    m = np.mod(t, 4294967296.0)
    m = np.where(m >= 2147483648.0, m - 4294967296.0, m)
    return m.astype(np.int64).astype(np.int32)


def cast(X, to):
    """cpu cast.ts:12-52: `to` is an ONNX TensorProto.DataType; FLOAT(1) -> float32,
    UINT8(2) / INT32(6) / INT64(7) -> int32 (no clipping), anything else throws."""
    X = np.asarray(X)
    if to == 1:
        return X.astype(np.float32)
    if to in (2, 6, 7):
        return js_to_int32(X) if X.dtype != np.int32 else X.copy()
    raise RefThrows("Cast: converting to DataType %d is not yet supported" % to)
