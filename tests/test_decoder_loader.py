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
    ("window on the attention only", _edit_node("attention", 1,
                                                lambda g, n: n["attrs"].update(window=16)),
     "declares another window"),
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


# Layers that differ the way a Gemma-4-style decoder's do
# (tools/export-recipes/gemma4/export_decode.py:59-82,510-527): sliding layers (head dim 32,
# window 8) and full layers (head dim 64); layers 3 and 4 share the K / V of the last owner of
# their kind (2 -> sliding layer 0... here: layer 3 reads layer 1, layer 4 reads layer 2).
MIXED = LlamaConfig(layers=5, d_model=256, ffn=384, heads=8, kv_heads=2, head_dim=32, vocab=512,
                    group_size=128, max_position=64,
                    layer_windows=(8, 8, 0, 8, 0), layer_head_dims=(32, 32, 64, 32, 64),
                    layer_kv_source=(0, 1, 2, 1, 2))


@pytest.fixture(scope="module")
def mixed_weights():
    return random_weights(MIXED, seed=21)


def test_round_trip_of_layers_that_differ(mixed_weights):
    """Per-layer window, head dim (with its RoPE tables) and KV source survive the file."""
    model = ka.open_model(decoder_model_file(mixed_weights))
    # q, o, gate, up, down everywhere; k and v in the three owners; the head
    assert len(ka.i4_resident_initializers(model)) == 5 * 5 + 2 * 3 + 1
    got = DecoderWeights.from_model(model)
    assert got.config == MIXED
    assert set(got.rope_by_depth) == {64}
    for depth in (32, 64):
        for a, b in zip(got.rope_of(depth), mixed_weights.rope_of(depth)):
            assert np.array_equal(a, b) and a.shape == (64, depth)
    for li, (a, b) in enumerate(zip(got.layers, mixed_weights.layers)):
        assert set(a) == set(b), li
        assert ("k" in a) == (MIXED.owner_of(li) == li)
        for name in a:
            if name.endswith("norm"):
                assert np.array_equal(a[name], b[name])
            else:
                assert np.array_equal(a[name].packed, b[name].packed), (li, name)


def _append_before_last_reader(graph):
    """Move the appends of layer 1's slots in front of layer 3's attention (their last reader)."""
    nodes = graph["nodes"]
    moved = [n for n in nodes if n["op"] == "state_append" and n["states"]["slot"].startswith("l1.")]
    rest = [n for n in nodes if n not in moved]
    first = next(i for i, n in enumerate(rest) if n["op"] == "attention" and n["outs"] == ["l3.att"])
    graph["nodes"] = rest[:first] + moved + rest[first:]


def _sharer_reads_other_rows(graph):
    att = next(n for n in graph["nodes"] if n["op"] == "attention" and n["outs"] == ["l3.att"])
    att["ins"][2] = "l0.v"     # v rows of another layer than its k rows


def _sharer_other_slots(graph):
    att = next(n for n in graph["nodes"] if n["op"] == "attention" and n["outs"] == ["l3.att"])
    att["states"] = {"k": "l0.k", "v": "l0.v"}


def _sharer_other_window(graph):
    att = next(n for n in graph["nodes"] if n["op"] == "attention" and n["outs"] == ["l3.att"])
    att["attrs"]["window"] = 16


def _appended_twice(graph):
    extra = next(n for n in graph["nodes"] if n["op"] == "state_append")
    graph["nodes"].append(dict(extra))


@pytest.mark.parametrize("name,edit,message", [
    ("append before the last reader", _append_before_last_reader, "before its last reader"),
    ("k and v of different layers", _sharer_reads_other_rows, "different layers"),
    ("another layer's slots", _sharer_other_slots, "roped rows and state slots"),
    ("another window than the owner", _sharer_other_window, "another head dim or window"),
    ("a slot appended twice", _appended_twice, "appended twice"),
])
def test_kv_sharing_graphs_that_break_the_rules_are_rejected(mixed_weights, name, edit, message):
    model = ka.open_model(decoder_model_file(mixed_weights, edit))
    with pytest.raises(GraphShapeError, match=message):
        DecoderWeights.from_model(model)


def test_config_rejects_inconsistent_layer_structure():
    base = dict(layers=3, d_model=64, ffn=64, heads=2, kv_heads=1, head_dim=32, vocab=16)
    with pytest.raises(ValueError, match="entries"):
        LlamaConfig(**base, layer_windows=(4, 4))
    with pytest.raises(ValueError, match="earlier layer"):
        LlamaConfig(**base, layer_kv_source=(0, 2, 2))          # a later layer
    with pytest.raises(ValueError, match="earlier layer"):
        LlamaConfig(**base, layer_kv_source=(0, 0, 1))          # layer 1 owns nothing itself
    with pytest.raises(ValueError, match="another head dim or window"):
        LlamaConfig(**base, layer_kv_source=(0, 0, 0), layer_windows=(4, 0, 4))
