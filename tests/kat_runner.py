"""Runs one known-answer case (tests/golden/kat.json) on the oracle or on the hip backend."""
import numpy as np

from util import arr


def _opt(case, key):
    return case.get(key)


def run_oracle(case):
    from oracle import ref

    op = case["op"]
    if op == "Gemm":
        C = arr(case["C"], case["C_shape"]) if case["C"] is not None else None
        return ref.gemm(arr(case["A"], case["A_shape"]), arr(case["B"], case["B_shape"]), C,
                        case["alpha"], case["beta"], case["transA"], case["transB"])
    if op == "MatMul":
        return ref.matmul(arr(case["A"], case["A_shape"]), arr(case["B"], case["B_shape"]))
    if op == "Conv":
        B = arr(case["B"], [len(case["B"])]) if case["B"] is not None else None
        return ref.conv(arr(case["X"], case["X_shape"]), arr(case["W"], case["W_shape"]), B,
                        case["dilations"], case["group"], None, case["pads"], case["strides"])
    if op == "MaxPool":
        return ref.maxpool(arr(case["X"], case["X_shape"]), case["kernel_shape"],
                           case.get("auto_pad", "NOTSET"), case.get("ceil_mode", 0),
                           _opt(case, "dilations"), _opt(case, "pads"), _opt(case, "strides"))
    if op == "Transpose":
        return ref.transpose(arr(case["X"], case["X_shape"]), case["perm"])
    if op in ("Add", "Sub", "Mul", "Div"):
        return ref.binary(op, arr(case["L"], case["L_shape"]), arr(case["R"], case["R_shape"]))
    if op == "GlobalAveragePool":
        return ref.global_average_pool(arr(case["X"], case["X_shape"]))
    if op == "Relu":
        return ref.unary("Relu", arr(case["X"], case["X_shape"]))
    if op == "Softmax":
        return ref.softmax(arr(case["X"], case["X_shape"]))
    if op == "LayerNormalization":
        return ref.layernorm_decomposed(arr(case["X"], case["X_shape"]), arr(case["gamma"], [-1]),
                                        arr(case["beta"], [-1]), case["epsilon"])
    raise KeyError(op)


def run_hip(ctx, case):
    from webdnn_amd import hostops as H

    up = lambda key, shape_key: ctx.move_tensor(arr(case[key], case[shape_key]))
    op = case["op"]
    if op == "Gemm":
        C = up("C", "C_shape") if case["C"] is not None else None
        y = H.gemm(ctx, up("A", "A_shape"), up("B", "B_shape"), C, case["alpha"], case["beta"],
                   case["transA"], case["transB"])
    elif op == "MatMul":
        y = H.matmul(ctx, up("A", "A_shape"), up("B", "B_shape"))
    elif op == "Conv":
        B = ctx.move_tensor(arr(case["B"], [len(case["B"])])) if case["B"] is not None else None
        y = H.conv(ctx, up("X", "X_shape"), up("W", "W_shape"), B, case["dilations"], case["group"],
                   None, case["pads"], case["strides"])
    elif op == "MaxPool":
        y = H.maxpool(ctx, up("X", "X_shape"), case["kernel_shape"], case.get("auto_pad", "NOTSET"),
                      case.get("ceil_mode", 0), _opt(case, "dilations"), _opt(case, "pads"),
                      _opt(case, "strides"))
    elif op == "Transpose":
        y = H.transpose(ctx, up("X", "X_shape"), case["perm"])
    elif op in ("Add", "Sub", "Mul", "Div"):
        y = H.binary(ctx, op, up("L", "L_shape"), up("R", "R_shape"))
    elif op == "GlobalAveragePool":
        y = H.global_average_pool(ctx, up("X", "X_shape"))
    elif op == "Relu":
        y = H.unary(ctx, "Relu", up("X", "X_shape"))
    elif op == "Softmax":
        y = H.softmax(ctx, up("X", "X_shape"))
    elif op == "LayerNormalization":
        y = H.layer_normalization(ctx, up("X", "X_shape"), ctx.move_tensor(arr(case["gamma"], [-1])),
                                  ctx.move_tensor(arr(case["beta"], [-1])), -1, case["epsilon"])
    else:
        raise KeyError(op)
    return y.get_data()


def expected(case):
    return arr(case["Y"], case["Y_shape"])


def case_id(case):
    keys = [k for k in ("A_shape", "B_shape", "X_shape", "W_shape", "L_shape", "R_shape") if k in case]
    return case["op"] + "-" + "x".join("_".join(map(str, case[k])) or "s" for k in keys)
