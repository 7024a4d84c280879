#!/usr/bin/env python3
"""Writes the model-archive fixtures of tests/golden/ with the protobuf library, not with this repository's own
writer: a check of the wire format that does not come from the code under test.

Runs in the build container only (needs /root/reference and google.protobuf).  The reference's message layout is
tfcc_runtime/proto/model.proto:1-91, common.proto:5-20, data.proto, operations/{base,math,nn}.proto; its generated
Python modules (tfcc_code_generator/backend/runtime/proto/*_pb2.py) carry each file's serialized descriptor as a bytes
literal.  Those modules are pre-protobuf-4 style and do not import under protobuf 7, and nothing of the reference is
imported or executed here: the files are read as text, the literal is taken out with `ast`, and the descriptors are
registered in a descriptor pool of this process.  The message classes the pool then hands out serialize one small
attention-shaped graph (MatmulWithBias, CreateVector, Reshape, Transpose, Matmul, Softmax, LayerNormalization), an
Inputs message and an Outputs message.  What is committed is message bytes and arrays - data - never the descriptors.

Outputs (all under tests/golden/):
  model_golden.zip            the archive as the reference's backend packs it: model.pb + model.npz
                              (tfcc_code_generator/backend/runtime/backend.py:37-49), weights through numpy.savez
  model_golden.pb             the same model.pb on its own, for a byte comparison with modelfile.py
  model_golden_inputs.pb      tfcc.runtime.data.Inputs for the test input
  model_golden_outputs.pb     tfcc.runtime.data.Outputs holding the float64-computed result rounded to fp32
  model_golden_arrays.npz     the test input, the weights and the expected output (float64 numpy model)
"""
import ast
import io
import os
import sys
import zipfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
REF = "/root/reference/tfcc_code_generator/backend/runtime/proto"

FLOAT, INT64 = 1, 7  # tfcc_runtime/proto/common.proto:5-20


def serialized_descriptor(path):
    """The bytes literal passed as serialized_pb= to FileDescriptor(...) in a generated *_pb2.py, read as text."""
    tree = ast.parse(open(path, encoding="utf-8").read())
    for node in ast.walk(tree):
        if isinstance(node, ast.Call) and getattr(node.func, "attr", getattr(node.func, "id", "")) == "FileDescriptor":
            for kw in node.keywords:
                if kw.arg == "serialized_pb":
                    call = kw.value  # _b('...')
                    arg = call.args[0] if isinstance(call, ast.Call) else call
                    value = ast.literal_eval(arg)
                    return value.encode("latin1") if isinstance(value, str) else value
    raise SystemExit("no serialized_pb in " + path)


def message_classes():
    from google.protobuf import any_pb2, descriptor_pb2, descriptor_pool, message_factory
    pool = descriptor_pool.DescriptorPool()
    pool.AddSerializedFile(any_pb2.DESCRIPTOR.serialized_pb)
    for rel in ("common_pb2.py", "model_pb2.py", "data_pb2.py", "operations/base_pb2.py", "operations/math_pb2.py",
                "operations/nn_pb2.py"):
        blob = serialized_descriptor(os.path.join(REF, rel))
        fd = descriptor_pb2.FileDescriptorProto.FromString(blob)  # parses: the literal is a whole descriptor
        pool.AddSerializedFile(fd.SerializeToString())
    get = lambda name: message_factory.GetMessageClass(pool.FindMessageTypeByName(name))
    return get, any_pb2.Any


def float64_model(x, w):
    """The graph below in float64."""
    x = x.astype(np.float64)
    q = x @ w["wq"].astype(np.float64) + w["bq"].astype(np.float64)      # [2, 6, 16]
    heads = q.reshape(2, 6, 4, 4).transpose(0, 2, 1, 3)                    # [2, 4, 6, 4]
    scores = heads @ heads.transpose(0, 1, 3, 2)                          # [2, 4, 6, 6]
    e = np.exp(scores - scores.max(axis=-1, keepdims=True))
    probs = e / e.sum(axis=-1, keepdims=True)
    ctx = (probs @ heads).transpose(0, 2, 1, 3).reshape(2, 6, 16)
    mean = ctx.mean(axis=-1, keepdims=True)
    var = ((ctx - mean) ** 2).mean(axis=-1, keepdims=True)
    return (ctx - mean) / np.sqrt(var + 1e-5) * w["gamma"].astype(np.float64) + w["beta"].astype(np.float64)


def main():
    get, Any = message_classes()
    Model, Graph, Symbol, Node = (get("tfcc.runtime.model." + n) for n in ("Model", "Graph", "Symbol", "Node"))
    ops = lambda n: get("tfcc.runtime.operations." + n)

    rng = np.random.default_rng(20211)
    weights = {"wq": rng.normal(0, 0.3, (16, 16)).astype(np.float32), "bq": rng.normal(0, 0.1, 16).astype(np.float32),
               "gamma": rng.normal(1, 0.1, 16).astype(np.float32), "beta": rng.normal(0, 0.1, 16).astype(np.float32)}
    x = rng.normal(size=(2, 6, 16)).astype(np.float32)

    g = Graph(name="golden")
    g.inputs.append("x")
    g.outputs.append("y")

    def symbol(name, dtype, kind, shape=None, ref=None):
        s = g.symbols.add(name=name, data_type=dtype)
        member = getattr(s, kind)
        member.SetInParent()
        if ref is not None:
            member.ref = ref
        if shape is not None:
            for d in shape:
                s.shape.dimensions.add(value=d)
        return name

    def node(name, op_message, inputs, outputs):
        n = g.nodes.add(name=name, version=1)
        n.inputs.extend(inputs)
        n.outputs.extend(outputs)
        n.operation.Pack(op_message)  # type.googleapis.com/<full name>, as Any::PackFrom (tfcc_runtime/utils/commutils.cpp:46-50)

    symbol("x", FLOAT, "view", [2, 6, 16])
    for ref in ("wq", "bq", "gamma", "beta"):
        symbol(ref, FLOAT, "constant_tensor", list(weights[ref].shape), ref)
    symbol("q", FLOAT, "variable")
    node("q_proj", ops("math.MatmulWithBias")(), ["x", "wq", "bq"], ["q"])
    symbol("shape_heads", INT64, "vector")
    cv = ops("base.CreateVector")(data_type=INT64)
    for d in (2, 6, 4, 4):
        cv.values.add(int64_value=d)
    node("shape_heads_make", cv, [], ["shape_heads"])
    symbol("q4", FLOAT, "view")
    node("split_heads", ops("base.Reshape")(), ["q", "shape_heads"], ["q4"])
    symbol("heads", FLOAT, "variable")
    node("heads_first", ops("base.Transpose")(perm=[0, 2, 1, 3]), ["q4"], ["heads"])
    symbol("heads_t", FLOAT, "variable")
    node("keys_transposed", ops("base.Transpose")(perm=[0, 1, 3, 2]), ["heads"], ["heads_t"])
    symbol("scores", FLOAT, "variable")
    node("scores_product", ops("math.Matmul")(), ["heads", "heads_t"], ["scores"])
    symbol("probs", FLOAT, "variable")
    node("scores_softmax", ops("math.Softmax")(axis=3), ["scores"], ["probs"])
    symbol("ctx", FLOAT, "variable")
    node("context_product", ops("math.Matmul")(), ["probs", "heads"], ["ctx"])
    symbol("ctx_t", FLOAT, "variable")
    node("heads_last", ops("base.Transpose")(perm=[0, 2, 1, 3]), ["ctx"], ["ctx_t"])
    symbol("shape_flat", INT64, "vector")
    cv2 = ops("base.CreateVector")(data_type=INT64)
    for d in (2, 6, 16):
        cv2.values.add(int64_value=d)
    node("shape_flat_make", cv2, [], ["shape_flat"])
    symbol("ctx_flat", FLOAT, "view")
    node("merge_heads", ops("base.Reshape")(), ["ctx_t", "shape_flat"], ["ctx_flat"])
    symbol("y", FLOAT, "variable")
    ln = ops("nn.LayerNormalization")()
    ln.epsilon.float_value = 1e-5
    node("norm", ln, ["ctx_flat", "gamma", "beta"], ["y"])

    model = Model(proto_version=1, name="golden_model", entrance_graph_name="golden")
    model.graphs.append(g)
    model_pb = model.SerializeToString(deterministic=True)

    DataItem = get("tfcc.runtime.data.DataItem")
    inputs = get("tfcc.runtime.data.Inputs")()
    inputs.items.add(name="x", dtype=FLOAT, shape=list(x.shape), data=x.tobytes())
    y64 = float64_model(x, weights)
    outputs = get("tfcc.runtime.data.Outputs")()
    outputs.items.add(name="y", dtype=FLOAT, shape=list(y64.shape), data=y64.astype(np.float32).tobytes())
    del DataItem

    npz = io.BytesIO()
    np.savez(npz, **{"golden/" + k: v for k, v in weights.items()})
    archive = io.BytesIO()
    with zipfile.ZipFile(archive, "w", zipfile.ZIP_STORED) as z:
        for name, blob in (("model.pb", model_pb), ("model.npz", npz.getvalue())):
            info = zipfile.ZipInfo(name, date_time=(2021, 1, 1, 0, 0, 0))  # fixed stamp: the fixture is reproducible
            z.writestr(info, blob)

    def write(name, blob):
        with open(os.path.join(HERE, name), "wb") as f:
            f.write(blob)
        print("%-28s %6d bytes" % (name, len(blob)))

    write("model_golden.zip", archive.getvalue())
    write("model_golden.pb", model_pb)
    write("model_golden_inputs.pb", inputs.SerializeToString(deterministic=True))
    write("model_golden_outputs.pb", outputs.SerializeToString(deterministic=True))
    arrays = io.BytesIO()
    np.savez(arrays, x=x, y64=y64, **weights)
    write("model_golden_arrays.npz", arrays.getvalue())


if __name__ == "__main__":
    if not os.path.isdir(REF):
        sys.exit("needs the reference tree at /root/reference (build container only)")
    main()
