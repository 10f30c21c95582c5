"""An independent evaluation of an ONNX-level graph (occamy_amd.compiler.Graph)
with torch CPU operators in float64 -- ONNX operator semantics written against
torch, sharing no code with the compiler, the executor or the oracle."""
import numpy as np
import torch
import torch.nn.functional as F


def evaluate(graph, inputs):
    env = {}
    for (name, _), a in zip(graph.input_shapes.items(), inputs):
        env[name] = torch.from_numpy(np.asarray(a))
        if env[name].dtype != torch.int64:
            env[name] = env[name].double()
    for name, a in graph.constants.items():
        t = torch.from_numpy(np.asarray(a))
        env[name] = t if t.dtype == torch.int64 else t.double()
    for op, ins, out, at in graph.nodes:
        x = [env[i] if i else None for i in ins]
        if op == "Conv":
            p = at.get("pads", [0, 0, 0, 0])
            env[out] = F.conv2d(x[0], x[1], x[2] if len(x) > 2 else None, stride=tuple(at.get("strides", [1, 1])),
                                padding=(p[0], p[1]), groups=at.get("group", 1))
        elif op == "Relu":
            env[out] = F.relu(x[0])
        elif op == "Sigmoid":
            env[out] = torch.sigmoid(x[0])
        elif op == "Tanh":
            env[out] = torch.tanh(x[0])
        elif op == "Clip":
            env[out] = torch.clamp(x[0], float(x[1]), float(x[2]))
        elif op == "Add":
            env[out] = x[0] + x[1]
        elif op == "Sub":
            env[out] = x[0] - x[1]
        elif op == "Mul":
            env[out] = x[0] * x[1]
        elif op == "Div":
            env[out] = x[0] / x[1]
        elif op == "Sqrt":
            env[out] = torch.sqrt(x[0])
        elif op == "Erf":
            env[out] = torch.erf(x[0])
        elif op == "Pow":
            env[out] = torch.pow(x[0], x[1])
        elif op == "Gelu":
            env[out] = F.gelu(x[0])
        elif op == "MaxPool":
            p = at.get("pads", [0, 0, 0, 0])
            env[out] = F.max_pool2d(x[0], tuple(at["kernel_shape"]), tuple(at.get("strides", [1, 1])), (p[0], p[1]))
        elif op == "AveragePool":
            p = at.get("pads", [0, 0, 0, 0])
            env[out] = F.avg_pool2d(x[0], tuple(at["kernel_shape"]), tuple(at.get("strides", [1, 1])), (p[0], p[1]),
                                    count_include_pad=True)
        elif op == "GlobalAveragePool":
            env[out] = x[0].mean((2, 3), keepdim=True)
        elif op == "ReduceMean":
            env[out] = x[0].mean(tuple(at["axes"]), keepdim=bool(at.get("keepdims", 1)))
        elif op == "Flatten":
            a = at.get("axis", 1)
            env[out] = x[0].reshape(int(np.prod(x[0].shape[:a])), -1)
        elif op == "Reshape":
            env[out] = x[0].reshape([int(v) for v in x[1]])
        elif op == "Transpose":
            env[out] = x[0].permute(*at["perm"])
        elif op == "Gather":
            env[out] = torch.index_select(x[0], at.get("axis", 0), x[1].reshape(-1)).reshape(
                tuple(x[0].shape[:at.get("axis", 0)]) + tuple(x[1].shape) + tuple(x[0].shape[at.get("axis", 0) + 1:]))
        elif op == "Softmax":
            env[out] = torch.softmax(x[0], at.get("axis", -1))
        elif op == "MatMul":
            env[out] = torch.matmul(x[0], x[1])
        elif op == "Gemm":
            a = x[0].T if at.get("transA", 0) else x[0]
            b = x[1].T if at.get("transB", 0) else x[1]
            env[out] = at.get("alpha", 1.0) * (a @ b) + (at.get("beta", 1.0) * x[2] if len(x) > 2 and x[2] is not None else 0)
        elif op == "LayerNormalization":
            env[out] = F.layer_norm(x[0], (x[0].shape[-1],), x[1], x[2], at.get("epsilon", 1e-5))
        elif op == "Cast":
            env[out] = x[0].double()
        elif op == "LeakyRelu":
            env[out] = F.leaky_relu(x[0], at.get("alpha", 0.01))
        elif op == "PRelu":
            env[out] = torch.where(x[0] < 0, x[0] * x[1], x[0])
        elif op == "Concat":
            env[out] = torch.cat(x, at["axis"])
        elif op == "Squeeze":
            if "axes" in at or len(x) > 1:
                axes = at["axes"] if "axes" in at else [int(v) for v in x[1]]
                env[out] = x[0].reshape([d for i, d in enumerate(x[0].shape) if i not in [a % x[0].dim() for a in axes]])
            else:
                env[out] = x[0].squeeze()
        elif op == "Unsqueeze":
            axes = at["axes"] if "axes" in at else [int(v) for v in x[1]]
            y = x[0]
            for a in sorted(a % (x[0].dim() + len(axes)) for a in axes):
                y = y.unsqueeze(a)
            env[out] = y
        elif op in ("Identity", "Dropout"):
            env[out] = x[0]
        elif op == "Expand":
            shape = torch.broadcast_shapes(tuple(x[0].shape), tuple(int(v) for v in x[1]))
            env[out] = x[0].expand(shape).contiguous()
        elif op == "Pad":
            assert all(int(v) == 0 for v in x[1]), "only the all-zero Pad is in the dialect's reach"
            env[out] = x[0]
        elif op == "BatchNormalization":
            env[out] = F.batch_norm(x[0], x[3], x[4], x[1], x[2], False, 0.0, at.get("epsilon", 1e-5))
        else:
            raise NotImplementedError(op)
    return [env[o].numpy() for o in graph.outputs]
