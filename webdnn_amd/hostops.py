"""Python host side of the hip backend: context, tensor and the hot-path operators.

Mirrors, for Python callers (tests, bench), what the Node.js host in
``webdnn_amd/js`` does for the descriptor runner: the same operator names,
attribute meaning and error behaviour as the reference's operator classes
(paths relative to src/descriptor_runner/ of the reference):

  HipContext / HipTensor   backend/wasm/wasmContextImpl.ts:13-163, wasmTensorImpl.ts:16-99
  shape logic              operators/base/{gemm,matmul,conv,maxpool,transpose,flatten,reshape5}.ts,
                           operators/operatorUtil.ts:169-245
  operator bodies          operators/cpu/operators/standard/*.ts (semantics), executed by the
                           HIP kernels behind include/webdnn_hip.h

All arithmetic happens on the GPU through the C ABI; nothing here computes
tensor values on the host, and there is no CPU fallback.
"""
import ctypes
import math

import numpy as np

from . import capi
from .capi import HipError, call

_DTYPES = {"float32": np.float32, "int32": np.int32}


class OperatorError(ValueError):
    """Raised where the reference operator throws (bad shapes / attributes)."""


def calc_strides(dims):
    """operators/operatorUtil.ts:169-176"""
    strides, length = [], 1
    for d in reversed(dims):
        strides.insert(0, length)
        length *= d
    return strides


def broadcast_uni(dims_a, dims_b):
    """operators/operatorUtil.ts:178-209: strides of B broadcast to A's shape."""
    if len(dims_a) < len(dims_b):
        raise OperatorError("Unidirectional broadcast error: %s, %s" % (dims_a, dims_b))
    expanded = [1] * (len(dims_a) - len(dims_b)) + list(dims_b)
    strides = calc_strides(expanded)
    for i, (a, b) in enumerate(zip(dims_a, expanded)):
        if a != b:
            if b == 1:
                strides[i] = 0
            else:
                raise OperatorError("Unidirectional broadcast error: %s, %s" % (dims_a, dims_b))
    return strides


def broadcast_multi(all_dims):
    """operators/operatorUtil.ts:211-245"""
    nd = max(len(d) for d in all_dims)
    expanded_all = [[1] * (nd - len(d)) + list(d) for d in all_dims]
    out = [max(e[i] for e in expanded_all) for i in range(nd)]
    all_strides = []
    for e in expanded_all:
        strides = calc_strides(e)
        for i in range(nd):
            if e[i] != out[i]:
                if e[i] == 1:
                    strides[i] = 0
                else:
                    raise OperatorError("Multidirectional broadcasting error: %s" % (all_dims,))
        all_strides.append(strides)
    return out, all_strides


class HipTensor:
    """A device tensor: a buffer handle plus dims.  Aliases share the handle through a
    reference count, as WasmSharedBuffer does (backend/wasm/wasmTensorImpl.ts:16-84)."""

    backend = "hip"

    def __init__(self, context, dims, data_type="float32", shared=None):
        if data_type not in _DTYPES:
            raise OperatorError("HipTensor: dataType %s not supported" % data_type)
        self.context = context
        self.dims = [int(d) for d in dims]
        self.ndim = len(self.dims)
        self.strides = calc_strides(self.dims)
        self.length = int(np.prod(self.dims, dtype=np.int64)) if self.dims else 1
        self.data_type = data_type
        if shared is None:
            handle = capi.load().wdh_alloc(self.length * 4)
            if handle == 0:
                raise HipError("wdh_alloc", -3, capi.last_error())
            shared = {"handle": handle, "refs": 0}
        self._shared = shared
        shared["refs"] += 1
        self._disposed = False

    @property
    def handle(self):
        if self._disposed:
            raise OperatorError("HipTensor used after dispose()")
        return self._shared["handle"]

    def alias(self, dims):
        """A tensor with other dims over the same buffer (zero-copy reshape)."""
        dims = [int(d) for d in dims]
        if (int(np.prod(dims, dtype=np.int64)) if dims else 1) != self.length:
            raise OperatorError("alias: element count differs")
        return HipTensor(self.context, dims, self.data_type, self._shared)

    def set_data(self, array):
        array = np.asarray(array, dtype=_DTYPES[self.data_type], order="C")
        if array.size != self.length:
            raise OperatorError("setData: length mismatch")
        call("wdh_write", self.handle, 0, array.ctypes.data_as(ctypes.c_void_p), array.nbytes)

    def get_data(self):
        out = np.empty(self.dims, dtype=_DTYPES[self.data_type])
        call("wdh_read", self.handle, 0, out.ctypes.data_as(ctypes.c_void_p), out.nbytes)
        return out

    def dispose(self):
        if self._disposed:
            return
        self._disposed = True
        self._shared["refs"] -= 1
        if self._shared["refs"] == 0:
            call("wdh_free", self._shared["handle"])


class HipContext:
    """backend/wasm/wasmContextImpl.ts:13-111 for the hip backend."""

    backend = "hip"

    def __init__(self, device=0):
        self.device = device
        self.initialized = False

    def initialize(self):
        call("wdh_init", self.device)
        self.initialized = True
        return self

    def device_info(self):
        name = ctypes.create_string_buffer(64)
        cu, mhz, hbm = ctypes.c_int(), ctypes.c_int(), ctypes.c_uint64()
        call("wdh_device_info", name, 64, ctypes.byref(cu), ctypes.byref(mhz), ctypes.byref(hbm))
        return {"name": name.value.decode(), "compute_units": cu.value, "clock_mhz": mhz.value,
                "hbm_bytes": hbm.value}

    def set_option(self, name, value):
        call("wdh_set_option", name.encode(), int(value))

    FORMS = ("gemm, B k-contiguous", "gemm, B n-contiguous", "conv, gathered taps", "conv, gathered taps (32-63)",
             "conv, gathered taps (flat loads)", "conv 1x1, X in place", "conv 3x3, LDS tile",
             "conv 7x7 s2 stem, weights and patch in LDS", "conv 1x1 stride 2, X in place", "conv 3x3, F(2x2,3x3) transforms + batched product",
             "conv 3x3, F(4x4,3x3) transforms + batched product")

    def last_plan(self):
        """Layout of the most recent Gemm / Conv launch: tile, whole tiles, tiles cut along K, chunks, form."""
        bm, bn, split, form = (ctypes.c_int() for _ in range(4))
        whole, cut = ctypes.c_int64(), ctypes.c_int64()
        call("wdh_last_plan", ctypes.byref(bm), ctypes.byref(bn), ctypes.byref(whole), ctypes.byref(cut),
             ctypes.byref(split), ctypes.byref(form))
        return {"tile": "%dx%d" % (bm.value, bn.value), "whole_tiles": whole.value, "split_tiles": cut.value,
                "split": split.value, "form": self.FORMS[form.value]}

    def empty_tensor(self, dims, data_type="float32"):
        return HipTensor(self, dims, data_type)

    def move_tensor(self, array):
        """CPU (numpy) -> hip, like moveTensor = emptyTensor + setData."""
        array = np.asarray(array)
        if array.dtype == np.float32:
            dt = "float32"
        elif array.dtype == np.int32:
            dt = "int32"
        else:
            raise OperatorError("moveTensor: dtype %s not supported" % array.dtype)
        t = self.empty_tensor(array.shape, dt)
        t.set_data(array)
        return t

    def sync(self):
        call("wdh_sync")

    def set_lane(self, lane):
        """wdh_set_lane: 0 = the default stream, 1 = the second one (recorded work and transfers only)."""
        call("wdh_set_lane", lane)

    def mem_stats(self):
        a, b, c = ctypes.c_uint64(), ctypes.c_uint64(), ctypes.c_uint64()
        call("wdh_mem_stats", ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
        return {"in_use": a.value, "cached": b.value, "peak": c.value}

    # captured runs (wdh_graph_*): record the device work between begin and end once, replay it
    def graph_begin(self):
        call("wdh_graph_begin")

    def graph_end(self):
        gid = ctypes.c_int(-1)
        call("wdh_graph_end", ctypes.byref(gid))
        return gid.value

    def graph_launch(self, graph_id):
        call("wdh_graph_launch", graph_id)

    def graph_destroy(self, graph_id):
        call("wdh_graph_destroy", graph_id)

    def event_record(self, idx):
        call("wdh_event_record", idx)

    def event_elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        call("wdh_event_elapsed_ms", a, b, ctypes.byref(ms))
        return ms.value


def _require_f32(*tensors):
    for t in tensors:
        if t is not None and t.data_type != "float32":
            raise OperatorError("only float32 is supported")


EPI = {None: 0, "relu": 1}


def gemm(ctx, a, b, c=None, alpha=1.0, beta=1.0, trans_a=0, trans_b=0, epilogue=None):
    """Gemm: operators/base/gemm.ts:28-61 + cpu gemm.ts:21-61."""
    _require_f32(a, b, c)
    if a.ndim != 2 or b.ndim != 2:
        raise OperatorError("Gemm: inputs must be 2-D")
    if trans_a:
        k, m = a.dims
        sa = (1, m)
    else:
        m, k = a.dims
        sa = (k, 1)
    if trans_b:
        n, kcheck = b.dims
        sb = (1, kcheck)
    else:
        kcheck, n = b.dims
        sb = (n, 1)
    if k != kcheck:
        raise OperatorError("Gemm: inner dimensions differ")
    sc = (0, 0)
    if c is not None:
        sc = broadcast_uni([m, n], c.dims)
    y = ctx.empty_tensor([m, n])
    call("wdh_gemm", a.handle, b.handle, c.handle if c is not None else 0, y.handle, 1, m, n, k,
         0, sa[0], sa[1], 0, sb[0], sb[1], sc[0], sc[1], alpha, beta, EPI[epilogue], 0)
    return y


def matmul_shape(dims_a, dims_b):
    """operators/base/matmul.ts:6-91"""
    if len(dims_a) == 0 or len(dims_b) == 0:
        raise OperatorError("MatMul: scalar input")
    total = max(len(dims_a), len(dims_b), 2)
    ea = list(dims_a)
    if len(ea) == 1:
        ea.insert(0, 1)
    ea = [1] * (total - len(ea)) + ea
    eb = list(dims_b)
    if len(eb) == 1:
        eb.append(1)
    eb = [1] * (total - len(eb)) + eb
    inner = ea[-1]
    if inner != eb[-2]:
        raise OperatorError("MatMul: inner dimensions differ")
    sa, sb = calc_strides(ea), calc_strides(eb)
    result = [ea[-2], eb[-1]]
    for i in range(total - 3, -1, -1):
        if ea[i] == 1:
            sa[i] = 0
        if eb[i] == 1:
            sb[i] = 0
        result.insert(0, max(ea[i], eb[i]))
    squeezed = list(result)
    if len(dims_a) == 1:
        del squeezed[-2]
    if len(dims_b) == 1:
        del squeezed[-1]
    return result, squeezed, sa, sb, inner


def matmul(ctx, a, b, bias=None, residual=None, epilogue=None):
    """MatMul: cpu matmul.ts:11-111 (result rank 2 or 3 only).  `bias` ([n]), `residual`
    (result-shaped) and `epilogue` express the fused MatMul+Add(+Relu) forms."""
    _require_f32(a, b, bias, residual)
    result, squeezed, sa, sb, inner = matmul_shape(a.dims, b.dims)
    if len(result) == 2:
        batch, m, n = 1, result[0], result[1]
        sab = sbb = 0
    elif len(result) == 3:
        batch, m, n = result
        sab, sbb = sa[0], sb[0]
    else:
        raise OperatorError("MatMul: result rank >= 4 is not supported")
    # a batch that only broadcasts B (stride 0) over dense A rows is one tall GEMM
    if (batch > 1 and sbb == 0 and sab == m * sa[-2] and residual is None
            and (bias is None or bias.ndim <= 1)):
        m, batch, sab = m * batch, 1, 0
    sc = (0, 0)
    if bias is not None:
        sc = broadcast_uni([m, n], bias.dims)
    y = ctx.empty_tensor(squeezed)
    call("wdh_gemm", a.handle, b.handle, bias.handle if bias is not None else 0, y.handle,
         batch, m, n, inner, sab, sa[-2], sa[-1], sbb, sb[-2], sb[-1], sc[0], sc[1], 1.0, 1.0,
         EPI[epilogue], residual.handle if residual is not None else 0)
    return y


def conv_shape(dims_x, dims_w, dilations=None, group=1, kernel_shape=None, pads=None, strides=None):
    """operators/base/conv.ts:31-79"""
    dilations = list(dilations) if dilations else [1, 1]
    kernel_shape = list(kernel_shape) if kernel_shape else [dims_w[2], dims_w[3]]
    pads = list(pads) if pads else [0, 0, 0, 0]
    strides = list(strides) if strides else [1, 1]
    in_shape = [dims_x[2], dims_x[3]]
    out_shape = [
        math.floor((in_shape[a] + pads[a] + pads[a + 2] - dilations[a] * (kernel_shape[a] - 1) - 1)
                   / strides[a]) + 1
        for a in range(2)
    ]
    return {"batch": dims_x[0], "dilations": dilations, "group": group, "kernel_shape": kernel_shape,
            "pads": pads, "strides": strides, "in_shape": in_shape, "out_shape": out_shape,
            "ch_in": dims_x[1], "ch_out": dims_w[0]}


def conv(ctx, x, w, b=None, dilations=None, group=1, kernel_shape=None, pads=None, strides=None,
         epilogue=None, residual=None, constant_weights=False):
    """Conv: cpu conv.ts:134-221; 2-D only.  constant_weights: `w` is not written to while it lives (what the
    runner says of an initializer's device copy), so the library may keep forms derived from it."""
    _require_f32(x, w, b, residual)
    if x.ndim != 4:
        raise OperatorError("Conv other than 2D is not yet supported")
    s = conv_shape(x.dims, w.dims, dilations, group, kernel_shape, pads, strides)
    y = ctx.empty_tensor([s["batch"], s["ch_out"], s["out_shape"][0], s["out_shape"][1]])
    call("wdh_conv2d_ex", x.handle, w.handle, b.handle if b is not None else 0, y.handle,
         s["batch"], s["ch_in"], s["in_shape"][0], s["in_shape"][1], s["ch_out"],
         s["kernel_shape"][0], s["kernel_shape"][1], s["pads"][0], s["pads"][1], s["pads"][2],
         s["pads"][3], s["strides"][0], s["strides"][1], s["dilations"][0], s["dilations"][1],
         group, EPI[epilogue], residual.handle if residual is not None else 0, 1 if constant_weights else 0)
    return y


_BIN = {"Add": 0, "Sub": 1, "Mul": 2, "Div": 3, "Pow": 4}


def binary(ctx, op, lhs, rhs):
    """Add/Sub/Mul/Div/Pow: cpu binary7.ts:16-68."""
    if lhs.data_type != rhs.data_type:
        raise OperatorError("Binary: input dataTypes mismatch: %s !== %s" % (lhs.data_type, rhs.data_type))
    out_shape, (sl, sr) = broadcast_multi([lhs.dims, rhs.dims])
    if len(out_shape) > 6:
        raise OperatorError("Binary: input ndim %d > 6 is not supported" % len(out_shape))
    if op == "Pow" and lhs.data_type != "float32":
        raise OperatorError("Pow: int32 is not supported on hip")
    y = ctx.empty_tensor(out_shape, lhs.data_type)
    nd = len(out_shape)
    shape_arr = (ctypes.c_int32 * max(nd, 1))(*out_shape)
    sl_arr = (ctypes.c_int64 * max(nd, 1))(*sl)
    sr_arr = (ctypes.c_int64 * max(nd, 1))(*sr)
    call("wdh_binary", _BIN[op], 0 if lhs.data_type == "float32" else 1, lhs.handle, rhs.handle,
         y.handle, nd, shape_arr, sl_arr, sr_arr)
    return y


_UN = {"Relu": 0, "Sigmoid": 1, "Sqrt": 2, "Exp": 3, "Tanh": 4, "Abs": 5, "Neg": 6, "Reciprocal": 7}
_UN_INT_OK = {"Relu", "Abs", "Neg"}


def unary(ctx, op, x):
    """cpu unary.ts:10-32"""
    if x.data_type != "float32" and op not in _UN_INT_OK:
        raise OperatorError("Unary: DataType %s not supported" % x.data_type)
    y = ctx.empty_tensor(x.dims, x.data_type)
    call("wdh_unary", _UN[op], 0 if x.data_type == "float32" else 1, x.handle, y.handle, x.length)
    return y


def softmax(ctx, x, axis=-1):
    """cpu softmax.ts:21-58: last axis only."""
    _require_f32(x)
    if axis < 0:
        axis += x.ndim
    if axis != x.ndim - 1:
        raise OperatorError("Softmax: currently only reducing final axis is supported")
    y = ctx.empty_tensor(x.dims)
    length = x.dims[axis]
    call("wdh_softmax", x.handle, y.handle, x.length // length if length else 0, length)
    return y


def linear_group(ctx, problems, epilogue=None):
    """Independent linear layers in as few launches as possible: problems = [(a [m,k], w [k,n], bias [n] or None)],
    returns the list of results.  Each is what gemm(a, w, bias) returns."""
    count = len(problems)
    ys, hs = [], {"a": [], "w": [], "b": [], "y": []}
    ms, ns, ks = [], [], []
    for a, w, b in problems:
        _require_f32(a, w, b)
        if a.ndim != 2 or w.ndim != 2 or a.dims[1] != w.dims[0] or (b is not None and list(b.dims) != [w.dims[1]]):
            raise OperatorError("linear_group: shapes %s %s %s" % (a.dims, w.dims, None if b is None else b.dims))
        y = ctx.empty_tensor([a.dims[0], w.dims[1]])
        ys.append(y)
        hs["a"].append(a.handle); hs["w"].append(w.handle); hs["b"].append(b.handle if b is not None else 0)
        hs["y"].append(y.handle)
        ms.append(a.dims[0]); ns.append(w.dims[1]); ks.append(a.dims[1])
    arr64 = lambda v: (ctypes.c_int64 * count)(*v)
    arr32 = lambda v: (ctypes.c_int32 * count)(*v)
    call("wdh_linear_group", count, arr64(hs["a"]), arr64(hs["w"]), arr64(hs["b"]), arr64(hs["y"]),
         arr32(ms), arr32(ns), arr32(ks), EPI[epilogue])
    return ys


def attention(ctx, q, k, v, heads, alpha):
    """softmax(alpha * Q_h K_h^T) V_h for every head h, heads side by side as in a
    [tokens, heads * d] projection: q [tq, heads*d], k and v [tk, heads*d] -> [tq, heads*d].
    The chain the reference runs node by node (cpu matmul.ts:11-111, softmax.ts:34-57)."""
    _require_f32(q, k, v)
    if q.ndim != 2 or k.ndim != 2 or v.ndim != 2:
        raise OperatorError("attention: q, k, v must be [tokens, heads*d]")
    width = q.dims[1]
    if heads <= 0 or width % heads or k.dims[1] != width or v.dims[1] != width or k.dims[0] != v.dims[0]:
        raise OperatorError("attention: shapes %s %s %s do not hold %d heads" % (q.dims, k.dims, v.dims, heads))
    d = width // heads
    y = ctx.empty_tensor(q.dims)
    call("wdh_attention", q.handle, k.handle, v.handle, y.handle, heads, q.dims[0], k.dims[0], d,
         d, width, d, width, d, width, d, width, float(alpha))
    return y


def layer_normalization(ctx, x, scale=None, bias=None, axis=-1, epsilon=1e-5):
    """ONNX LayerNormalization (opset 17) over the last axis."""
    _require_f32(x, scale, bias)
    if axis < 0:
        axis += x.ndim
    if axis != x.ndim - 1:
        raise OperatorError("LayerNormalization: only the last axis is supported")
    length = x.dims[-1]
    for t in (scale, bias):
        if t is not None and t.length != length:
            raise OperatorError("LayerNormalization: scale/bias must have the normalised length")
    y = ctx.empty_tensor(x.dims)
    call("wdh_layernorm", x.handle, scale.handle if scale is not None else 0,
         bias.handle if bias is not None else 0, y.handle, x.length // length if length else 0,
         length, epsilon)
    return y


def layer_normalization_add(ctx, x, scale, bias, addend, axis=-1, epsilon=1e-5):
    """LayerNormalization and the Add that follows it: returns (normalised, normalised + addend),
    addend of x's shape.  One launch for the node pair."""
    _require_f32(x, scale, bias, addend)
    if axis < 0:
        axis += x.ndim
    if axis != x.ndim - 1:
        raise OperatorError("LayerNormalization: only the last axis is supported")
    if list(addend.dims) != list(x.dims):
        raise OperatorError("LayerNormalization+Add: the addend must have the input's shape")
    length = x.dims[-1]
    for t in (scale, bias):
        if t is not None and t.length != length:
            raise OperatorError("LayerNormalization: scale/bias must have the normalised length")
    y, y2 = ctx.empty_tensor(x.dims), ctx.empty_tensor(x.dims)
    call("wdh_layernorm_add", x.handle, scale.handle if scale is not None else 0,
         bias.handle if bias is not None else 0, y.handle, addend.handle, y2.handle,
         x.length // length if length else 0, length, epsilon)
    return y, y2


def reduce_mean_last(ctx, x, keepdims=1):
    """ReduceMean over the last axis: cpu reduce.ts:369-405."""
    _require_f32(x)
    length = x.dims[-1]
    out_dims = x.dims[:-1] + ([1] if keepdims else [])
    y = ctx.empty_tensor(out_dims)
    call("wdh_reduce_mean", x.handle, y.handle, x.length // length if length else 0, length)
    return y


def reduce_mean(ctx, x, axes=(), keepdims=1):
    """ReduceMean over any axes (all of them when `axes` is empty): cpu reduce.ts:40-131, 369-405 --
    one pass per axis in ascending order, fp32 between the passes, the last pass divides by the
    product of the reduced extents."""
    _require_f32(x)
    nd = x.ndim
    ax = sorted(int(a) + nd if int(a) < 0 else int(a) for a in axes) if len(axes) else list(range(nd))
    if any(not 0 <= a < nd for a in ax) or len(set(ax)) != len(ax):
        raise OperatorError("ReduceMean: axes out of range or repeated")
    shape, cur, total = list(x.dims), x, 1
    for i, a in enumerate(ax):
        red = shape[a]
        total *= red
        outer, inner = int(np.prod(shape[:a], dtype=np.int64)), int(np.prod(shape[a + 1:], dtype=np.int64))
        shape[a] = 1
        nxt = ctx.empty_tensor(shape)
        call("wdh_reduce_axis", cur.handle, nxt.handle, outer, red, inner, total if i == len(ax) - 1 else 1)
        if cur is not x:
            cur.dispose()
        cur = nxt
    if cur is x:                                   # rank 0: nothing to reduce
        return x.alias(list(x.dims))
    if not keepdims:
        out = cur.alias([d for i, d in enumerate(shape) if i not in ax])
        cur.dispose()
        return out
    return cur


def maxpool_shape(dims_x, kernel_shape, auto_pad="NOTSET", ceil_mode=0, dilations=None, pads=None,
                  strides=None):
    """operators/base/maxpool.ts:32-137"""
    dilations = list(dilations) if dilations else [1, 1]
    strides = list(strides) if strides else [1, 1]
    in_shape = [dims_x[2], dims_x[3]]
    if auto_pad == "NOTSET":
        pads = list(pads) if pads else [0, 0, 0, 0]
        rnd = math.ceil if ceil_mode else math.floor
        out_shape = [
            rnd((in_shape[a] + pads[a] + pads[a + 2] - dilations[a] * (kernel_shape[a] - 1) - 1)
                / strides[a]) + 1
            for a in range(2)
        ]
    elif auto_pad in ("SAME_UPPER", "SAME_LOWER"):
        out_shape = [math.ceil(in_shape[a] / strides[a]) for a in range(2)]
        total = [(out_shape[a] - 1) * strides[a] + ((kernel_shape[a] - 1) * dilations[a] + 1)
                 - in_shape[a] for a in range(2)]
        lo = [math.floor(t / 2) for t in total]
        hi = [math.ceil(t / 2) for t in total]
        pads = lo + hi if auto_pad == "SAME_UPPER" else hi + lo
    elif auto_pad == "VALID":
        out_shape = [math.ceil((in_shape[a] - dilations[a] * (kernel_shape[a] - 1)) / strides[a])
                     for a in range(2)]
        pads = [0, 0, 0, 0]
    else:
        raise OperatorError("Unknown auto_pad %s for MaxPool" % auto_pad)
    return {"dilations": dilations, "strides": strides, "pads": pads, "in_shape": in_shape,
            "out_shape": out_shape}


def maxpool(ctx, x, kernel_shape, auto_pad="NOTSET", ceil_mode=0, dilations=None, pads=None,
            strides=None, storage_order=0, n_outputs=1):
    """MaxPool: cpu maxpool.ts:12-56."""
    _require_f32(x)
    if storage_order != 0:
        raise OperatorError("MaxPool: storage_order !== 0 is not supported.")
    if n_outputs != 1:
        raise OperatorError("MaxPool: output indices is not yet supported")
    if x.ndim != 4:
        raise OperatorError("MaxPool other than 2D is not yet supported")
    s = maxpool_shape(x.dims, kernel_shape, auto_pad, ceil_mode, dilations, pads, strides)
    if s["pads"][0] < 0 or s["pads"][1] < 0:
        raise OperatorError("MaxPool: negative padding")
    y = ctx.empty_tensor([x.dims[0], x.dims[1], s["out_shape"][0], s["out_shape"][1]])
    call("wdh_maxpool2d", x.handle, y.handle, x.dims[0], x.dims[1], x.dims[2], x.dims[3],
         s["out_shape"][0], s["out_shape"][1], kernel_shape[0], kernel_shape[1], s["pads"][0],
         s["pads"][1], s["strides"][0], s["strides"][1], s["dilations"][0], s["dilations"][1])
    return y


def global_average_pool(ctx, x):
    """cpu globalaveragepool.ts:12-41"""
    _require_f32(x)
    if x.ndim != 4:
        raise OperatorError("GlobalAveragePool other than 2D is not yet supported")
    y = ctx.empty_tensor([x.dims[0], x.dims[1], 1, 1])
    call("wdh_global_avgpool", x.handle, y.handle, x.dims[0] * x.dims[1], x.dims[2] * x.dims[3])
    return y


def transpose(ctx, x, perm=None):
    """operators/base/transpose.ts:16-34 + cpu transpose.ts:12-44."""
    perm = list(perm) if perm else [x.ndim - 1 - i for i in range(x.ndim)]
    if len(perm) != x.ndim:
        raise OperatorError("Transpose: perm length differs from rank")
    if x.ndim < 1 or x.ndim > 6:
        raise OperatorError("Transpose: ndim %d is not supported" % x.ndim)
    out_shape = [x.dims[p] for p in perm]
    in_strides = [x.strides[p] for p in perm]
    y = ctx.empty_tensor(out_shape, x.data_type)
    shape_arr = (ctypes.c_int32 * x.ndim)(*out_shape)
    stride_arr = (ctypes.c_int64 * x.ndim)(*in_strides)
    call("wdh_transpose", x.handle, y.handle, x.ndim, shape_arr, stride_arr)
    return y


def flatten(ctx, x, axis=1):
    """operators/base/flatten.ts:7-17; shares the input buffer like cpu flatten.ts:11-20."""
    if axis != 1:
        raise OperatorError("Flatten: only axis === 1 is supported")
    rest = int(np.prod(x.dims[1:], dtype=np.int64)) if x.ndim > 1 else 1
    return x.alias([x.dims[0], rest])


def reshape_shape(dims, length, shape_input, allowzero=False):
    """operators/base/reshape5.ts:16-75"""
    explicit, minus = 1, -1
    for i, s in enumerate(shape_input):
        if s > 0:
            explicit *= s
        elif s == 0 and not allowzero:
            explicit *= dims[i]
        elif s == 0:
            pass
        else:
            if s != -1 and not allowzero:
                raise OperatorError("Reshape: negative dimension")
            if s == -1:
                if minus >= 0:
                    raise OperatorError("Reshape: multiple -1 dimensions")
                minus = i
    if minus >= 0 and explicit <= 0:
        raise OperatorError("Reshape: cannot infer -1")
    out = []
    for i, s in enumerate(shape_input):
        if s > 0 or (s == 0 and allowzero):
            out.append(s)
        elif s == 0:
            out.append(dims[i])
        else:
            out.append(length // explicit)
    return out


def reshape(ctx, x, shape_input, allowzero=False):
    """Reshape (opset >= 5): the shape tensor lives on the CPU (a list here); zero-copy alias."""
    return x.alias(reshape_shape(x.dims, x.length, [int(s) for s in shape_input], allowzero))


def gather(ctx, data, indices, axis=0):
    """Gather along `axis` with an int32 index tensor of any rank."""
    if indices.data_type != "int32":
        raise OperatorError("Gather: indices must be int32")
    if axis < 0:
        axis += data.ndim
    if not 0 <= axis < data.ndim:
        raise OperatorError("Gather: axis out of range")
    outer = int(np.prod(data.dims[:axis], dtype=np.int64))
    inner = int(np.prod(data.dims[axis + 1:], dtype=np.int64))
    out_dims = data.dims[:axis] + indices.dims + data.dims[axis + 1:]
    y = ctx.empty_tensor(out_dims, data.data_type)
    call("wdh_gather", data.handle, indices.handle, y.handle, outer, data.dims[axis], inner,
         indices.length)
    return y


# ---- layout glue on the device --------------------------------------------------------

def _dense_strides(dims):
    out, acc = [], 1
    for d in reversed(dims):
        out.insert(0, acc)
        acc *= d
    return out


def _strided_copy(x, x_offset, y, y_offset, shape, x_strides, y_strides):
    nd = len(shape)
    if nd > 6:
        raise OperatorError("strided copy: rank %d is not supported" % nd)
    call("wdh_strided_copy", x.handle, x_offset, y.handle, y_offset, nd,
         (ctypes.c_int32 * max(nd, 1))(*shape), (ctypes.c_int64 * max(nd, 1))(*x_strides),
         (ctypes.c_int64 * max(nd, 1))(*y_strides))


def squeeze_shape(dims, axes):
    """operators/base/squeeze.ts:8-22"""
    if not axes:
        return [s for s in dims if s != 1]
    nn = [a if a >= 0 else a + len(dims) for a in axes]
    return [s for i, s in enumerate(dims) if i not in nn]


def squeeze(ctx, x, axes=()):
    """Squeeze (both the attribute and the input-tensor form of `axes`): zero-copy alias,
    as cpu squeeze.ts:12-37 shares the input buffer."""
    shape = squeeze_shape(x.dims, [int(a) for a in axes])
    if int(np.prod(shape, dtype=np.int64)) != x.length:
        raise OperatorError("Squeeze: removed axis is not of extent 1")
    return x.alias(shape)


def unsqueeze_shape(dims, axes):
    """operators/base/unsqueeze.ts:8-27"""
    nd = len(dims) + len(axes)
    nn = [a if a >= 0 else a + nd for a in axes]
    shape, src = [], 0
    for d in range(nd):
        if d in nn:
            shape.append(1)
        else:
            if src >= len(dims):
                raise OperatorError("Unsqueeze: axes out of range")
            shape.append(dims[src])
            src += 1
    if src != len(dims):
        raise OperatorError("Unsqueeze: duplicate axes")
    return shape


def unsqueeze(ctx, x, axes):
    return x.alias(unsqueeze_shape(x.dims, [int(a) for a in axes]))


def concat(ctx, inputs, axis=0):
    """cpu concat.ts:21-84: one strided copy per input into its band of the output."""
    first = inputs[0]
    ax = axis if axis >= 0 else first.ndim + axis
    if ax < 0 or ax >= first.ndim:
        raise OperatorError("Concat: axis %d out of range" % ax)
    for t in inputs:
        if t.ndim != first.ndim or any(t.dims[d] != first.dims[d] for d in range(first.ndim) if d != ax):
            raise OperatorError("Concat: input shapes differ outside the axis")
        if t.data_type != first.data_type:
            raise OperatorError("Concat: input data types differ")
    out_shape = list(first.dims)
    out_shape[ax] = sum(t.dims[ax] for t in inputs)
    y = ctx.empty_tensor(out_shape, first.data_type)
    ys = _dense_strides(out_shape)
    offset = 0
    for t in inputs:
        if t.length:
            _strided_copy(t, 0, y, offset * ys[ax], t.dims, _dense_strides(t.dims), ys)
        offset += t.dims[ax]
    return y


def split(ctx, x, n_outputs, axis=0, split=()):
    """operators/base/split.ts:10-70 + cpu split.ts:12-45"""
    ax = axis if axis >= 0 else axis + x.ndim
    if ax < 0 or ax >= x.ndim:
        raise OperatorError("Split: axis %d out of range" % ax)
    parts = [int(s) for s in split] if len(split) else [x.dims[ax] // n_outputs] * n_outputs
    if len(parts) < n_outputs or any(p < 0 for p in parts) or sum(parts[:n_outputs]) > x.dims[ax]:
        raise OperatorError("Split: parts do not fit the axis")
    xs = _dense_strides(x.dims)
    outs, offset = [], 0
    for n in range(n_outputs):
        shape = list(x.dims)
        shape[ax] = parts[n]
        y = ctx.empty_tensor(shape, x.data_type)
        if y.length:
            _strided_copy(x, offset * xs[ax], y, 0, shape, xs, _dense_strides(shape))
        outs.append(y)
        offset += parts[n]
    return outs


def slice_ranges(dims, starts, ends, axes=None, steps=None):
    """cpu slice.ts:19-58: per axis (start, step, extent of the result), with the reference's
    clamping (start to [0, size-1], stop to [-1, size])."""
    nd = len(dims)
    if nd > 6:
        raise OperatorError("Slice: input dimension %d > 6 is not yet supported" % nd)
    if axes is not None:
        axes = [int(a) + nd if int(a) < 0 else int(a) for a in axes]
    else:
        axes = list(range(nd))
    steps = [int(s) for s in steps] if steps is not None else [1] * len(axes)
    ranges = [[0, d, 1] for d in dims]
    for i, a in enumerate(axes):
        if not 0 <= a < nd:
            raise OperatorError("Slice: axis out of range")
        if steps[i] == 0:
            raise OperatorError("Slice: step 0")
        ranges[a] = [int(starts[i]), int(ends[i]), steps[i]]
    out = []
    for (start, stop, step), size in zip(ranges, dims):
        if start < 0:
            start += size
        start = max(min(start, size - 1), 0)
        if stop < 0:
            stop += size
        stop = max(min(stop, size), -1)
        out.append((start, step, max(-((start - stop) // step), 0)))  # ceil((stop-start)/step)
    return out


def slice_(ctx, x, starts, ends, axes=None, steps=None):
    """Slice (opset >= 10); starts/ends/axes/steps live on the CPU (lists here)."""
    r = slice_ranges(x.dims, starts, ends, axes, steps)
    shape = [n for (_, _, n) in r]
    y = ctx.empty_tensor(shape, x.data_type)
    if y.length:
        xs = _dense_strides(x.dims)
        _strided_copy(x, sum(st * s for (st, _, _), s in zip(r, xs)), y, 0, shape,
                      [step * s for (_, step, _), s in zip(r, xs)], _dense_strides(shape))
    return y


_CAST_TO = {1: "float32", 2: "int32", 6: "int32", 7: "int32"}


def cast(ctx, x, to):
    """cpu cast.ts:12-52 (`to` is an ONNX TensorProto.DataType)."""
    if to not in _CAST_TO:
        raise OperatorError("Cast: converting to DataType %d is not yet supported" % to)
    dt = _CAST_TO[to]
    y = ctx.empty_tensor(x.dims, dt)
    call("wdh_cast", 0 if x.data_type == "float32" else 1, 0 if dt == "float32" else 1,
         x.handle, y.handle, x.length)
    return y
