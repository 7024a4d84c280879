"""One post-LayerNorm transformer encoder layer composed from the CPU oracle's functions
(oracle_lib: sgemm with double accumulation, softmax, layer_norm, gelu_accurate), node for node
the graph that modelfile.bert_encoder_layer writes.  Test infrastructure only."""
import numpy as np

import oracle_lib as O


def encoder_layer(x, w, heads, epsilon=1e-12, mask=None):
    batch, seq, hidden = x.shape
    size = hidden // heads
    x2 = x.reshape(batch * seq, hidden)

    def project(name_w, name_b):
        return O.sgemm(x2, w[name_w], w[name_b]).reshape(batch, seq, heads, size)

    q = np.ascontiguousarray(project("wq", "bq").transpose(0, 2, 1, 3))
    kt = np.ascontiguousarray(project("wk", "bk").transpose(0, 2, 3, 1))
    v = np.ascontiguousarray(project("wv", "bv").transpose(0, 2, 1, 3))
    scores = O.sgemm(q, kt) / np.float32(np.sqrt(size))
    if mask is not None:  # [batch, 1, 1, seq], added to every head's and every query's scores
        scores = scores.astype(np.float32) + mask.astype(np.float32)
    probs = O.softmax(scores.astype(np.float32))
    context = np.ascontiguousarray(O.sgemm(probs, v).transpose(0, 2, 1, 3)).reshape(batch * seq, hidden)
    attention = O.layer_norm(O.sgemm(context, w["wo"], w["bo"]) + x2, w["ln1_gamma"], w["ln1_beta"], epsilon)
    inner = O.gelu_accurate(O.sgemm(attention, w["w1"], w["b1"]))
    out = O.layer_norm(O.sgemm(inner, w["w2"], w["b2"]) + attention, w["ln2_gamma"], w["ln2_beta"], epsilon)
    return out.reshape(batch, seq, hidden)
