"""Interprets a graph written by webdnn_amd.modelgen with the C oracle (oracle/ref.py),
node by node, the way the reference's runner would with its CPU operators."""
import numpy as np

from oracle import ref


def run_graph(model, feeds, keep=None):
    """model: webdnn_amd.modelgen.parse_model(...) result; feeds: {input name: array}.
    Returns {output name: array} (plus every tensor named in `keep`)."""
    # the runner clips INT64 tensors to int32 when it loads them (core/runnerImpl.ts:167-198)
    to32 = lambda v: v.astype(np.int32) if isinstance(v, np.ndarray) and v.dtype == np.int64 else v
    env = {k: to32(v) for k, v in model["initializers"].items()}
    env.update(feeds)
    for n in model["nodes"]:
        x = [env[i] for i in n["inputs"]]
        a = n["attrs"]
        op = n["op_type"]
        if op == "Gemm":
            y = ref.gemm(x[0], x[1], x[2] if len(x) > 2 else None, a.get("alpha", 1.0), a.get("beta", 1.0),
                         a.get("transA", 0), a.get("transB", 0))
        elif op == "MatMul":
            y = ref.matmul(x[0], x[1])
        elif op == "Conv":
            y = ref.conv(x[0], x[1], x[2] if len(x) > 2 else None, a.get("dilations"), a.get("group", 1),
                         a.get("kernel_shape"), a.get("pads"), a.get("strides"))
        elif op in ("Add", "Sub", "Mul", "Div", "Pow"):
            y = ref.binary(op, x[0], x[1])
        elif op in ("Relu", "Sigmoid", "Sqrt", "Exp", "Tanh", "Abs", "Neg", "Reciprocal"):
            y = ref.unary(op, x[0])
        elif op == "Softmax":
            y = ref.softmax(x[0], a.get("axis", -1))
        elif op == "MaxPool":
            y = ref.maxpool(x[0], a["kernel_shape"], a.get("auto_pad", "NOTSET"), a.get("ceil_mode", 0),
                            a.get("dilations"), a.get("pads"), a.get("strides"))
        elif op == "GlobalAveragePool":
            y = ref.global_average_pool(x[0])
        elif op == "Flatten":
            y = ref.flatten(x[0], a.get("axis", 1))
        elif op == "Reshape":
            y = ref.reshape(x[0], x[1], a.get("allowzero", 0))
        elif op == "Transpose":
            y = ref.transpose(x[0], a.get("perm"))
        elif op == "LayerNormalization":
            y = ref.layernorm_decomposed(x[0], x[1] if len(x) > 1 else None, x[2] if len(x) > 2 else None,
                                         a.get("epsilon", 1e-5))
        elif op == "ReduceMean":
            y = ref.reduce_mean(x[0], a.get("axes", []), a.get("keepdims", 1))
        elif op == "Squeeze":
            y = ref.squeeze(x[0], x[1].reshape(-1) if len(x) > 1 else a.get("axes", []))
        elif op == "Unsqueeze":
            y = ref.unsqueeze(x[0], x[1].reshape(-1) if len(x) > 1 else a.get("axes", []))
        elif op == "Concat":
            y = ref.concat(x, a.get("axis", 0))
        elif op == "Split":
            parts = x[1].reshape(-1) if len(x) > 1 else a.get("split", [])
            for name, part in zip(n["outputs"], ref.split(x[0], len(n["outputs"]), a.get("axis", 0), parts)):
                env[name] = part
            continue
        elif op == "Slice":
            y = ref.slice_(x[0], x[1], x[2], x[3] if len(x) > 3 else None, x[4] if len(x) > 4 else None)
        elif op == "Cast":
            y = ref.cast(x[0], a.get("to", 1))
        elif op == "Constant":
            y = to32(a["value"])
        elif op == "Shape":
            y = np.array(x[0].shape, np.int32)
        elif op == "Gather":
            y = ref.gather(x[0], x[1], a.get("axis", 0))
        else:
            raise NotImplementedError(op)
        env[n["outputs"][0]] = np.asarray(y)
    out = {name: env[name] for name, _ in model["outputs"]}
    for name in keep or []:
        out[name] = env[name]
    return out
