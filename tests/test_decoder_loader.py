"""Model file -> decoder weights, on the CPU: a small decoder written out as a Karume model
file (tests/model_file.py, the decode recipe's node order) comes back with every array and the
whole config intact, and graphs that are valid IR but not the decoder shape this backend runs
are rejected by name."""
import numpy as np
import pytest

import karume_amd as ka
from karume_amd.decoder import DecoderWeights, LlamaConfig, random_weights
from karume_amd.decoder_loader import GraphShapeError
from model_file import decoder_model_file

SMALL = LlamaConfig(layers=2, d_model=256, ffn=384, heads=8, kv_heads=2, head_dim=32, vocab=512,
                    group_size=128, max_position=64)


@pytest.fixture(scope="module")
def weights():
    return random_weights(SMALL, seed=12)


def test_round_trip_keeps_every_array_and_the_config(weights):
    model = ka.open_model(decoder_model_file(weights))
    assert len(ka.i4_resident_initializers(model)) == 7 * SMALL.layers + 1
    got = DecoderWeights.from_model(model)
    assert got.config == SMALL          # rope_base is not in a file; the tables are
    assert np.array_equal(got.embedding, weights.embedding) and got.embedding.dtype == np.float16
    assert np.array_equal(got.rope_cos, weights.rope_cos)
    assert np.array_equal(got.rope_sin, weights.rope_sin)
    assert np.array_equal(got.final_norm, weights.final_norm)
    for a, b in zip(got.layers, weights.layers):
        assert set(a) == set(b)
        for name in ("attn_norm", "ffn_norm"):
            assert np.array_equal(a[name], b[name]) and a[name].dtype == np.float32
        for name in ("q", "k", "v", "o", "gate", "up", "down"):
            assert (a[name].n, a[name].k) == (b[name].n, b[name].k), name
            assert np.array_equal(a[name].packed, b[name].packed), name
            # the file carries f32 scale companions (docs/ir-v1.md:135-150)
            assert a[name].scales.dtype == np.float32
            assert np.array_equal(a[name].scales, b[name].scales.astype(np.float32)), name
    assert np.array_equal(got.lm_head.packed, weights.lm_head.packed)


def _edit_node(op, index, fn):
    def edit(graph):
        nodes = [n for n in graph["nodes"] if n["op"] == op]
        fn(graph, nodes[index])
    return edit


def _drop_append(graph):
    graph["nodes"] = [n for n in graph["nodes"]
                      if not (n["op"] == "state_append" and n["states"]["slot"] == "l1.v")]


def _rope_on_v(graph):
    att = [n for n in graph["nodes"] if n["op"] == "attention"][0]
    att["ins"][2] = att["ins"][1]           # v reads the roped k


def _f32_linear(graph):
    graph["initializers"]["l0.o_proj"]["storage"] = {"dtype": "f32"}


@pytest.mark.parametrize("name,edit,message", [
    ("sliding window", _edit_node("attention", 1, lambda g, n: n["attrs"].update(window=16)),
     "sliding-window"),
    ("two eps", _edit_node("rms_norm", 2, lambda g, n: n["attrs"].update(eps=1e-6)), "uniform"),
    ("other scale", _edit_node("attention", 0, lambda g, n: n["attrs"].update(scale=0.5)),
     "uniform|attention scale"),
    ("KV-sharing layer", _drop_append, "state_append"),
    ("rope on v", _rope_on_v, "RoPE is expected on q and k and not on v"),
    ("plain attention", _edit_node("attention", 0, lambda g, n: n.pop("states")), "states form"),
    ("no argmax", lambda g: g["nodes"].pop(), "argmax"),
])
def test_graphs_outside_the_decoder_shape_are_rejected_by_name(weights, name, edit, message):
    model = ka.open_model(decoder_model_file(weights, edit))
    with pytest.raises(GraphShapeError, match=message):
        DecoderWeights.from_model(model)


def test_a_linear_that_is_not_int4_or_has_a_bias_is_rejected(weights):
    def f32_o_proj(tensors):
        out = []
        for key, dtype, shape, data in tensors:
            if key == "l0.o_proj":
                out.append((key, "F32", shape, np.zeros(shape, dtype="<f4").tobytes()))
            elif key == "karume.scale.l0.o_proj":
                continue
            else:
                out.append((key, dtype, shape, data))
        return out

    model = ka.open_model(decoder_model_file(weights, _f32_linear, f32_o_proj))
    with pytest.raises(GraphShapeError, match="int4-resident"):
        DecoderWeights.from_model(model)

    def biased(tensors):
        return [(k, t, s, np.ones(s, dtype="<f4").tobytes() if k == "l1.down_proj.bias" else d)
                for k, t, s, d in tensors]

    model = ka.open_model(decoder_model_file(weights, None, biased))
    with pytest.raises(GraphShapeError, match="not all zeros"):
        DecoderWeights.from_model(model)
