"""The model wire format against fixtures that were written by the protobuf library from the reference's own
message descriptors (tests/golden/make_model_golden.py), not by this repository's writer:
  - modelfile.py must emit the same bytes for the same graph, the same Inputs message, and read the Outputs message;
  - the runtime must load the archive (its own zip / npz / wire readers) and compute the float64 model's result."""
import io
import os
import zipfile

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _read(name):
    with open(os.path.join(GOLDEN, name), "rb") as f:
        return f.read()


@pytest.fixture(scope="module")
def mf(pkg):
    import importlib
    return importlib.import_module("wechat_tfcc_amd.modelfile")


def _same_graph_with_the_repository_writer(mf, arrays):
    g = mf.GraphBuilder("golden")
    g.input("x", mf.FLOAT, [2, 6, 16])
    for ref in ("wq", "bq", "gamma", "beta"):
        g.constant(ref, arrays[ref])
    V, W, VEC = mf.VARIABLE, mf.VIEW, mf.VECTOR
    g._symbol("q", mf.FLOAT, V)
    g.node("math.MatmulWithBias", ["x", "wq", "bq"], ["q"], name="q_proj")
    g._symbol("shape_heads", mf.INT64, VEC)
    make = lambda dims: b"".join(mf.f_bytes(1, mf.f_varint(1, d)) for d in dims) + mf.f_varint(2, mf.INT64)
    g.node("base.CreateVector", [], ["shape_heads"], make((2, 6, 4, 4)), name="shape_heads_make")
    g._symbol("q4", mf.FLOAT, W)
    g.node("base.Reshape", ["q", "shape_heads"], ["q4"], name="split_heads")
    g._symbol("heads", mf.FLOAT, V)
    g.node("base.Transpose", ["q4"], ["heads"], mf.f_packed(1, [0, 2, 1, 3]), name="heads_first")
    g._symbol("heads_t", mf.FLOAT, V)
    g.node("base.Transpose", ["heads"], ["heads_t"], mf.f_packed(1, [0, 1, 3, 2]), name="keys_transposed")
    g._symbol("scores", mf.FLOAT, V)
    g.node("math.Matmul", ["heads", "heads_t"], ["scores"], name="scores_product")
    g._symbol("probs", mf.FLOAT, V)
    g.node("math.Softmax", ["scores"], ["probs"], mf.f_varint(1, 3), name="scores_softmax")
    g._symbol("ctx", mf.FLOAT, V)
    g.node("math.Matmul", ["probs", "heads"], ["ctx"], name="context_product")
    g._symbol("ctx_t", mf.FLOAT, V)
    g.node("base.Transpose", ["ctx"], ["ctx_t"], mf.f_packed(1, [0, 2, 1, 3]), name="heads_last")
    g._symbol("shape_flat", mf.INT64, VEC)
    g.node("base.CreateVector", [], ["shape_flat"], make((2, 6, 16)), name="shape_flat_make")
    g._symbol("ctx_flat", mf.FLOAT, W)
    g.node("base.Reshape", ["ctx_t", "shape_flat"], ["ctx_flat"], name="merge_heads")
    g._symbol("y", mf.FLOAT, V)
    g.node("nn.LayerNormalization", ["ctx_flat", "gamma", "beta"], ["y"], mf.f_bytes(1, mf.value_message(1e-5)), name="norm")
    g.output("y")
    return g


def test_writer_emits_the_bytes_the_protobuf_library_emits(mf):
    arrays = np.load(io.BytesIO(_read("model_golden_arrays.npz")))
    g = _same_graph_with_the_repository_writer(mf, arrays)
    archive = mf.write_model([g], "golden", name="golden_model")
    with zipfile.ZipFile(io.BytesIO(archive)) as z:
        mine = z.read("model.pb")
    want = _read("model_golden.pb")
    assert mine == want
    # the archive fixture holds the same message
    with zipfile.ZipFile(io.BytesIO(_read("model_golden.zip"))) as z:
        assert z.read("model.pb") == want
        assert sorted(z.namelist()) == ["model.npz", "model.pb"]
    assert mf.encode_inputs({"x": arrays["x"]}) == _read("model_golden_inputs.pb")
    got = mf.decode_outputs(_read("model_golden_outputs.pb"))
    assert list(got) == ["y"] and got["y"].dtype == np.float32
    assert np.array_equal(got["y"], arrays["y64"].astype(np.float32))


@pytest.mark.gpu
def test_runtime_loads_the_golden_archive_and_matches_the_float64_model(pkg, dev, mf):
    import importlib
    rt = importlib.import_module("wechat_tfcc_amd.runtime_api")
    arrays = np.load(io.BytesIO(_read("model_golden_arrays.npz")))
    model = rt.Model(_read("model_golden.zip"))
    # the Inputs message as the protobuf library wrote it goes to the runtime untouched
    out = mf.decode_outputs(model.run_serialized(_read("model_golden_inputs.pb")))
    assert list(out) == ["y"] and out["y"].shape == (2, 6, 16)
    want = arrays["y64"]
    err = np.linalg.norm(out["y"].astype(np.float64) - want) / np.linalg.norm(want)
    assert err <= 1e-5, err
    # ... and the Outputs message the runtime serializes reads back with the same fields the library writes
    again = model.run({"x": arrays["x"]})["y"]
    assert np.array_equal(again, out["y"])
    model.close()
