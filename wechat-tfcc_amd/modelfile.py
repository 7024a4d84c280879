"""Writer of the runtime's model archive and of its input / output messages, in pure Python.

A model archive is a zip with `model.pb` (tfcc.runtime.model.Model, proto3) and `model.npz` (the
constants, keyed "<graph name>/<ref>"): tfcc_runtime/framework/model.cpp:57-80, written in the
reference by tfcc_code_generator/backend/runtime/backend.py:37-49 and modelgenerator.py:33-41.
Field numbers are those of tfcc_runtime/proto/model.proto, common.proto, data.proto and
operations/{math,base,nn}.proto; the encoding is the public protobuf wire format, produced here
directly so that no protobuf package or generated module is needed.

`bert_encoder_layer` lays out one post-LayerNorm transformer encoder layer the way the reference's
converter lowers it: MatmulWithBias for the six projections, Reshape + Transpose around the two
batched Matmul nodes, Div by sqrt(head size), Softmax, Gelu, Add + LayerNormalization.
"""
import io
import struct
import zipfile

import numpy as np

FLOAT, UINT8, INT8, UINT16, INT16, INT32, INT64, BOOL, DOUBLE, UINT32, UINT64 = 1, 2, 3, 4, 5, 6, 7, 9, 11, 12, 13
NP_OF = {FLOAT: np.float32, UINT8: np.uint8, INT8: np.int8, UINT16: np.uint16, INT16: np.int16, INT32: np.int32,
         INT64: np.int64, BOOL: np.uint8, DOUBLE: np.float64, UINT32: np.uint32, UINT64: np.uint64}
DTYPE_OF = {np.dtype(v): k for k, v in NP_OF.items() if k != BOOL}

VARIABLE, VIEW, CONSTANT_TENSOR, VALUE, CONSTANT_VALUE, VECTOR, CONSTANT_VECTOR = 3, 4, 5, 6, 7, 8, 9


# ---- wire format ---------------------------------------------------------------------------------
def _varint(v):
    v &= (1 << 64) - 1
    out = bytearray()
    while v >= 0x80:
        out.append((v & 0x7F) | 0x80)
        v >>= 7
    out.append(v)
    return bytes(out)


def f_varint(field, v):
    return _varint(field << 3) + _varint(v)


def f_bytes(field, payload):
    if isinstance(payload, str):
        payload = payload.encode()
    return _varint(field << 3 | 2) + _varint(len(payload)) + bytes(payload)


def f_float(field, v):
    return _varint(field << 3 | 5) + struct.pack("<f", v)


def f_double(field, v):
    return _varint(field << 3 | 1) + struct.pack("<d", v)


def f_packed(field, values):
    return f_bytes(field, b"".join(_varint(v) for v in values)) if len(values) else b""


def read_fields(buf):
    """Yields (field, wire type, value) of one message; value is int or bytes."""
    pos, n = 0, len(buf)

    def varint():
        nonlocal pos
        v, shift = 0, 0
        while True:
            b = buf[pos]
            pos += 1
            v |= (b & 0x7F) << shift
            if not b & 0x80:
                return v
            shift += 7

    while pos < n:
        key = varint()
        field, wt = key >> 3, key & 7
        if wt == 0:
            yield field, wt, varint()
        elif wt == 2:
            ln = varint()
            yield field, wt, bytes(buf[pos:pos + ln])
            pos += ln
        elif wt == 5:
            yield field, wt, bytes(buf[pos:pos + 4])
            pos += 4
        elif wt == 1:
            yield field, wt, bytes(buf[pos:pos + 8])
            pos += 8
        else:
            raise ValueError("unsupported wire type %d" % wt)


# ---- data.proto ------------------------------------------------------------------------------------
def encode_inputs(arrays):
    """{name: ndarray} -> serialized tfcc.runtime.data.Inputs"""
    out = b""
    for name, a in arrays.items():
        a = np.ascontiguousarray(a)
        item = f_bytes(1, name) + f_varint(2, DTYPE_OF[a.dtype]) + f_packed(3, list(a.shape)) + f_bytes(4, a.tobytes())
        out += f_bytes(1, item)
    return out


def decode_outputs(buf):
    """serialized tfcc.runtime.data.Outputs -> {name: ndarray}"""
    result = {}
    for field, wt, item in read_fields(buf):
        if field != 2 or wt != 2:
            continue
        name, dtype, shape, data = "", 0, [], b""
        for f, t, v in read_fields(item):
            if f == 1:
                name = v.decode()
            elif f == 2:
                dtype = v
            elif f == 3 and t == 2:
                shape += _unpack(v)
            elif f == 3:
                shape.append(v)
            elif f == 4:
                data = v
        result[name] = np.frombuffer(data, dtype=NP_OF[dtype]).reshape(shape).copy()
    return result


def _unpack(packed):
    pos, out = 0, []
    while pos < len(packed):
        v, shift = 0, 0
        while True:
            b = packed[pos]
            pos += 1
            v |= (b & 0x7F) << shift
            if not b & 0x80:
                break
            shift += 7
        out.append(v)
    return out


# ---- model.proto -----------------------------------------------------------------------------------
def value_message(v, kind="float"):
    """tfcc.runtime.common.Value"""
    if kind == "float":
        return f_float(3, v)
    if kind == "double":
        return f_double(4, v)
    if kind == "int64":
        return f_varint(1, int(v))
    return f_varint(2, int(v))


def any_message(package_and_name, payload=b""):
    url = "type.googleapis.com/tfcc.runtime.operations." + package_and_name
    return f_bytes(1, url) + (f_bytes(2, payload) if payload else b"")


class GraphBuilder:
    def __init__(self, name):
        self.name = name
        self.inputs, self.outputs, self.symbols, self.nodes = [], [], [], []
        self.constants = {}
        self._n = 0

    def _symbol(self, name, dtype, kind, shape=None, ref=None):
        body = f_bytes(1, name) + f_varint(2, dtype) + f_bytes(kind, f_bytes(1, ref) if ref is not None else b"")
        if shape is not None:
            dims = b"".join(f_bytes(1, f_varint(1, d) if isinstance(d, int) else f_bytes(2, d)) for d in shape)
            body += f_bytes(10, dims)
        self.symbols.append(body)
        return name

    def fresh(self, stem):
        self._n += 1
        return "%s_%d" % (stem, self._n)

    def input(self, name, dtype, shape):
        self.inputs.append(name)
        return self._symbol(name, dtype, VIEW, shape)

    def value_input(self, name, dtype):
        self.inputs.append(name)
        return self._symbol(name, dtype, VALUE)

    def variable(self, stem, dtype=FLOAT, shape=None):
        return self._symbol(self.fresh(stem), dtype, VARIABLE, shape)

    def view(self, stem, dtype=FLOAT, shape=None):
        return self._symbol(self.fresh(stem), dtype, VIEW, shape)

    def value(self, stem, dtype=FLOAT):
        return self._symbol(self.fresh(stem), dtype, VALUE)

    def vector(self, stem, dtype=INT64):
        return self._symbol(self.fresh(stem), dtype, VECTOR)

    def constant(self, ref, array, kind=CONSTANT_TENSOR):
        array = np.asarray(array)
        self.constants["%s/%s" % (self.name, ref)] = array
        return self._symbol(ref, DTYPE_OF[array.dtype], kind, list(array.shape) if kind == CONSTANT_TENSOR else None, ref)

    def node(self, op, inputs, outputs, payload=b"", version=1, name=None):
        body = f_bytes(1, name or self.fresh(op.split(".")[-1].lower()))
        body += b"".join(f_bytes(2, i) for i in inputs) + b"".join(f_bytes(3, o) for o in outputs)
        body += f_bytes(4, any_message(op, payload)) + f_varint(5, version)
        self.nodes.append(body)

    def output(self, name):
        self.outputs.append(name)

    # -- operations ---------------------------------------------------------------------------------
    def matmul(self, a, b, bias=None):
        out = self.variable("matmul")
        if bias is None:
            self.node("math.Matmul", [a, b], [out])
        else:
            self.node("math.MatmulWithBias", [a, b, bias], [out])
        return out

    def binary(self, op, a, b):
        out = self.variable(op.lower())
        self.node("math." + op, [a, b], [out])
        return out

    def unary(self, op, a, payload=b""):
        out = self.variable(op.split(".")[-1].lower())
        self.node(op, [a], [out], payload)
        return out

    def softmax(self, a, axis):
        return self.unary("math.Softmax", a, f_varint(1, axis))

    def transpose(self, a, perm):
        return self.unary("base.Transpose", a, f_packed(1, perm))

    def layer_norm(self, a, gamma, beta, epsilon):
        out = self.variable("layernorm")
        self.node("nn.LayerNormalization", [a, gamma, beta], [out], f_bytes(1, value_message(epsilon)))
        return out

    def reshape(self, a, dims):
        """dims: 0 keeps the input's dimension, -1 is inferred"""
        shape = self.vector("shape", INT64)
        values = b"".join(f_bytes(1, f_varint(1, d)) for d in dims)
        self.node("base.CreateVector", [], [shape], values + f_varint(2, INT64))
        out = self.view("reshape")
        self.node("base.Reshape", [a, shape], [out])
        return out

    def serialize(self):
        body = f_bytes(1, self.name) + b"".join(f_bytes(2, i) for i in self.inputs)
        body += b"".join(f_bytes(3, o) for o in self.outputs)
        body += b"".join(f_bytes(4, s) for s in self.symbols) + b"".join(f_bytes(5, n) for n in self.nodes)
        return body


def write_model(graphs, entrance, name="model", userdata=None, compress=False):
    """-> bytes of the model archive"""
    pb = f_varint(1, 1) + f_bytes(2, name) + b"".join(f_bytes(3, g.serialize()) for g in graphs) + f_bytes(4, entrance)
    constants = {}
    for g in graphs:
        constants.update(g.constants)
    npz = io.BytesIO()
    if constants:
        (np.savez_compressed if compress else np.savez)(npz, **constants)
    else:
        with zipfile.ZipFile(npz, "w"):
            pass
    out = io.BytesIO()
    with zipfile.ZipFile(out, "w", zipfile.ZIP_DEFLATED if compress else zipfile.ZIP_STORED) as z:
        z.writestr("model.pb", pb)
        z.writestr("model.npz", npz.getvalue())
        if userdata is not None:
            z.writestr("userdata", userdata)
    return out.getvalue()


def bert_layer_weights(rng, hidden=768, ffn=3072, std=0.02):
    w = {}
    for name, shape in (("wq", (hidden, hidden)), ("wk", (hidden, hidden)), ("wv", (hidden, hidden)),
                        ("wo", (hidden, hidden)), ("w1", (hidden, ffn)), ("w2", (ffn, hidden))):
        w[name] = rng.normal(0, std, shape).astype(np.float32)
    for name, n in (("bq", hidden), ("bk", hidden), ("bv", hidden), ("bo", hidden), ("b1", ffn), ("b2", hidden)):
        w[name] = rng.normal(0, std, n).astype(np.float32)
    for name in ("ln1", "ln2"):
        w[name + "_gamma"] = (1 + rng.normal(0, std, hidden)).astype(np.float32)
        w[name + "_beta"] = rng.normal(0, std, hidden).astype(np.float32)
    return w


def bert_encoder_layer(weights, batch, seq, heads, epsilon=1e-12, graph_name="encoder", with_mask=False):
    """One encoder layer: input `hidden_states` [batch, seq, hidden] -> output `layer_output`.  with_mask: a second
    input `attention_mask` [batch, 1, 1, seq] is added to the divided scores before the softmax."""
    hidden = weights["wq"].shape[0]
    size = hidden // heads
    g = GraphBuilder(graph_name)
    x = g.input("hidden_states", FLOAT, [batch, seq, hidden])
    c = {k: g.constant(k, v) for k, v in weights.items()}
    scale = g.constant("attention_scale", np.array(np.sqrt(size), dtype=np.float32), CONSTANT_VALUE)

    def heads_of(t, perm):
        return g.transpose(g.reshape(t, [0, 0, heads, size]), perm)

    q = heads_of(g.matmul(x, c["wq"], c["bq"]), [0, 2, 1, 3])        # [b, h, s, d]
    kt = heads_of(g.matmul(x, c["wk"], c["bk"]), [0, 2, 3, 1])       # [b, h, d, s]
    v = heads_of(g.matmul(x, c["wv"], c["bv"]), [0, 2, 1, 3])
    scores = g.binary("Div", g.matmul(q, kt), scale)
    if with_mask:
        scores = g.binary("Add", scores, g.input("attention_mask", FLOAT, [batch, 1, 1, seq]))
    probs = g.softmax(scores, 3)
    context = g.reshape(g.transpose(g.matmul(probs, v), [0, 2, 1, 3]), [0, 0, hidden])
    attention = g.layer_norm(g.binary("Add", g.matmul(context, c["wo"], c["bo"]), x), c["ln1_gamma"], c["ln1_beta"],
                             epsilon)
    inner = g.unary("math.Gelu", g.matmul(attention, c["w1"], c["b1"]))
    out = g.layer_norm(g.binary("Add", g.matmul(inner, c["w2"], c["b2"]), attention), c["ln2_gamma"], c["ln2_beta"],
                       epsilon)
    # the graph's output keeps a stable name
    final = g._symbol("layer_output", FLOAT, VARIABLE, [batch, seq, hidden])
    g.node("base.Identity", [out], [final])
    g.output(final)
    return g
