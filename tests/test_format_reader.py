"""On-disk reader (safetensors + karume_ir weight table).  The cases restate the reference's
packages/runtime/tests/format_safetensors_test.ts and format_container_test.ts (weight-table
part) and open the data files its golden tests hold.  CPU only."""
import glob
import json
import os
import struct

import numpy as np
import pytest
from safetensors.numpy import load_file

import helpers
from helpers import oracle
from karume_amd.format_i4 import pack_int4
from karume_amd.format_model import (ContainerError, IrError, SafetensorsError,
                                     build_safetensors, i4_resident_initializers, open_model,
                                     packed_int4, parse_safetensors, tensor_bytes)


def raw_file(header: dict, data: bytes) -> bytes:
    """A file with exactly this header (no validation, 8-byte padded) — for malformed cases."""
    text = json.dumps(header).encode()
    text += b" " * (-(8 + len(text)) % 8)
    return struct.pack("<Q", len(text)) + text + data


def f32(values) -> bytes:
    return np.asarray(values, dtype="<f4").tobytes()


# ---- parse_safetensors: format_safetensors_test.ts:12-199 -------------------------------------

def test_tensor_table_and_metadata():
    buffer = build_safetensors([("a", "F32", [2, 2], f32([1, 2, 3, 4])),
                                ("b", "I32", [3], np.array([5, 6, 7], "<i4").tobytes())],
                               {"note": "hello"})
    file = parse_safetensors(buffer)
    assert file.metadata == {"note": "hello"}
    assert list(file.tensors) == ["a", "b"]
    a, b = file.tensors["a"], file.tensors["b"]
    assert (a.dtype, a.shape, a.byte_length) == ("F32", (2, 2), 16)
    assert np.frombuffer(tensor_bytes(file, a), "<f4").tolist() == [1, 2, 3, 4]
    assert np.frombuffer(tensor_bytes(file, b), "<i4").tolist() == [5, 6, 7]
    assert b.byte_offset == a.byte_offset + 16 and a.byte_offset % 8 == 0


def test_views_share_the_callers_buffer():
    buffer = bytearray(build_safetensors([("a", "F32", [1], f32([1.5]))]))
    file = parse_safetensors(buffer)
    view = file.tensors["a"]
    buffer[view.byte_offset:view.byte_offset + 4] = f32([-2.0])
    assert np.frombuffer(tensor_bytes(file, view), "<f4")[0] == -2.0


@pytest.mark.parametrize("blob, fragment", [
    (b"\x00" * 7, "too short"),
    (struct.pack("<Q", 100) + b"{}", "exceeds the file length"),
    (struct.pack("<Q", 2 ** 60) + b"{}", "exceeds the safe integer range"),
    (struct.pack("<Q", 8) + b"{not json", "cannot be parsed"),
    (struct.pack("<Q", 2) + b"\xff\xfe", "UTF-8"),
    (struct.pack("<Q", 2) + b"[]", "not an object"),
])
def test_broken_framing_is_rejected(blob, fragment):
    with pytest.raises(SafetensorsError, match=fragment):
        parse_safetensors(blob)


@pytest.mark.parametrize("header, size, fragment", [
    ({"a": {"dtype": "F64", "shape": [1], "data_offsets": [0, 8]}}, 8, "unsupported dtype"),
    ({"a": {"dtype": "F32", "shape": [3], "data_offsets": [0, 8]}}, 8, "size mismatch"),
    ({"a": {"dtype": "F32", "shape": [-1], "data_offsets": [0, 4]}}, 4, "non-negative integer"),
    ({"a": {"dtype": "F32", "shape": [1.5], "data_offsets": [0, 4]}}, 4, "non-negative integer"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4.5]}}, 4, "non-negative integer"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0]}}, 4, "2 needed"),
    ({"a": {"dtype": "F32", "shape": "x", "data_offsets": [0, 4]}}, 4, "shape is not an array"),
    ({"a": 3}, 0, "not an object"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}}, 4, "outside the data"),
    ({"a": {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]},
      "b": {"dtype": "F32", "shape": [1], "data_offsets": [4, 8]}}, 8, "overlaps"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]},
      "b": {"dtype": "F32", "shape": [1], "data_offsets": [8, 12]}}, 12, "unused bytes"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [0, 4]}}, 8, "unused bytes at the end"),
    ({"a": {"dtype": "I8", "shape": [1], "data_offsets": [0, 1]},
      "b": {"dtype": "F32", "shape": [1], "data_offsets": [1, 5]}}, 5, "not aligned"),
    ({"w": {"dtype": "I4", "shape": [3], "data_offsets": [0, 2]}}, 2, "byte boundary"),
    ({"a": {"dtype": "I8", "shape": [2], "data_offsets": [0, 2]},
      "w": {"dtype": "I4", "shape": [4], "data_offsets": [2, 4]}}, 4, "not aligned"),
    ({"__metadata__": {"k": 1}}, 0, "not a string"),
    ({"a": {"dtype": "F32", "shape": [1], "data_offsets": [8, 4]}}, 8, "reversed"),
])
def test_bad_declarations_are_rejected(header, size, fragment):
    with pytest.raises(SafetensorsError, match=fragment):
        parse_safetensors(raw_file(header, bytes(size)))


def test_i4_keeps_the_logical_shape_and_half_the_bytes():
    file = parse_safetensors(build_safetensors([("w", "I4", [3, 32], bytes(48))]))
    view = file.tensors["w"]
    assert view.shape == (3, 32) and view.byte_length == 48
    assert len(tensor_bytes(file, view)) == 48


def test_zero_sized_tensors_are_accepted():
    file = parse_safetensors(build_safetensors([("e", "F32", [0, 4], b""),
                                                ("a", "F32", [1], f32([1]))]))
    assert file.tensors["e"].byte_length == 0 and file.tensors["a"].byte_length == 4


def test_agrees_with_the_safetensors_library_on_every_golden_file():
    paths = sorted(glob.glob(os.path.join(helpers.GOLDEN, "*", "*.safetensors")))
    assert len(paths) >= 7
    for path in paths:
        with open(path, "rb") as handle:
            file = parse_safetensors(handle.read())
        want = load_file(path)
        assert set(file.tensors) == set(want)
        for name, view in file.tensors.items():
            assert view.shape == want[name].shape
            assert bytes(tensor_bytes(file, view)) == want[name].tobytes()


# ---- open_model: format_container_test.ts:23-260,463 ------------------------------------------

def base_graph() -> dict:
    return {
        "format": "karume-ir", "version": 1, "requires": {"ops": ["linear"]}, "symbols": [],
        "inputs": [{"name": "x", "dtype": "f32", "shape": [1, 4]}], "outputs": ["y"],
        "initializers": {"w": {"tensor": "enc.w", "storage": {"dtype": "f32"}},
                         "b": {"tensor": "enc.b", "storage": {"dtype": "f32"}}},
        "values": {"w": {"dtype": "f32", "shape": [3, 4]}, "b": {"dtype": "f32", "shape": [3]},
                   "y": {"dtype": "f32", "shape": [1, 3]}},
        "nodes": [{"op": "linear", "ins": ["x", "w", "b"], "outs": ["y"], "attrs": {}}],
    }


BASE_TENSORS = [("enc.w", "F32", [3, 4], f32([0.5] * 12)), ("enc.b", "F32", [3], f32([1, 2, 3]))]


def model_bytes(graph, tensors=None, metadata=True) -> bytes:
    meta = {"karume_ir": json.dumps(graph)} if metadata else None
    return build_safetensors(BASE_TENSORS if tensors is None else tensors, meta)


def i4_model(group=32, scale=("enc.w.scale", "F32", [4, 2], f32([1] * 8))):
    graph = base_graph()
    graph["values"]["w"] = {"dtype": "f32", "shape": [4, 64]}
    graph["values"]["b"] = {"dtype": "f32", "shape": [4]}
    graph["inputs"][0]["shape"] = [1, 64]
    graph["initializers"]["w"]["storage"] = {"dtype": "i4", "scale": "enc.w.scale",
                                             "group_size": group}
    tensors = [("enc.w", "I4", [4, 64], bytes(128)), scale,
               ("enc.b", "F32", [4], f32([1, 2, 3, 4]))]
    return graph, tensors


def test_open_model_joins_graph_and_tensors():
    model = open_model(model_bytes(base_graph()))
    assert set(model.initializers) == {"w", "b"}
    assert model.initializers["w"].tensor == "enc.w"
    assert model.initializers["w"].shape == (3, 4)
    assert model.graph["nodes"][0]["op"] == "linear"


def test_missing_graph_json_is_rejected():
    with pytest.raises(ContainerError, match="karume_ir"):
        open_model(model_bytes(base_graph(), metadata=False))


def test_missing_initializer_tensor_is_rejected():
    with pytest.raises(ContainerError, match="'enc.w' is not in the file"):
        open_model(model_bytes(base_graph(), BASE_TENSORS[1:]))


def test_storage_dtype_must_match_the_file():
    graph = base_graph()
    graph["initializers"]["w"]["storage"] = {"dtype": "f16"}
    with pytest.raises(ContainerError, match="needs F16"):
        open_model(model_bytes(graph))


def test_declared_shape_must_match_the_file():
    graph = base_graph()
    graph["values"]["w"] = {"dtype": "f32", "shape": [4, 3]}
    with pytest.raises(ContainerError, match="declared shape"):
        open_model(model_bytes(graph))


def test_semantic_and_storage_dtype_must_combine():
    graph = base_graph()
    graph["values"]["w"] = {"dtype": "i32", "shape": [3, 4]}
    with pytest.raises(IrError, match="cannot be combined"):
        open_model(model_bytes(graph))
    graph = base_graph()
    graph["initializers"]["w"]["storage"] = {"dtype": "i32"}
    with pytest.raises(IrError, match="cannot be combined"):
        open_model(model_bytes(graph))


def test_i32_initializer_is_matched_with_an_i32_tensor():
    graph = base_graph()
    graph["values"]["b"] = {"dtype": "i32", "shape": [3]}
    graph["initializers"]["b"]["storage"] = {"dtype": "i32"}
    tensors = [BASE_TENSORS[0], ("enc.b", "I32", [3], np.array([1, 2, 3], "<i4").tobytes())]
    assert open_model(model_bytes(graph, tensors)).initializers["b"].storage.dtype == "i32"
    with pytest.raises(ContainerError, match="needs I32"):
        open_model(model_bytes(graph))


def test_missing_scale_tensor_is_rejected():
    graph = base_graph()
    graph["initializers"]["w"]["storage"] = {"dtype": "i8", "scale": "enc.w.scale"}
    tensors = [("enc.w", "I8", [3, 4], bytes(12)), BASE_TENSORS[1]]
    with pytest.raises(ContainerError, match="scale tensor"):
        open_model(model_bytes(graph, tensors))


def test_unreferenced_tensors_are_all_listed_in_name_order():
    tensors = [BASE_TENSORS[0], ("enc.w_old", "F32", [3, 4], f32([1] * 12)), BASE_TENSORS[1],
               ("enc.dead", "F32", [2], f32([1, 2]))]
    with pytest.raises(ContainerError, match=r"\(2\): enc.dead, enc.w_old"):
        open_model(model_bytes(base_graph(), tensors))


def test_scale_tensors_count_as_referenced():
    graph = base_graph()
    graph["initializers"]["w"]["storage"] = {"dtype": "i8", "scale": "enc.w.scale"}
    tensors = [("enc.w", "I8", [3, 4], bytes(12)),
               ("enc.w.scale", "F32", [3, 1], f32([1, 1, 1])), BASE_TENSORS[1]]
    assert len(open_model(model_bytes(graph, tensors)).file.tensors) == 3
    # keepdim broadcast shape: same rank, every dim 1 or the weight's
    tensors[1] = ("enc.w.scale", "F32", [3], f32([1, 1, 1]))
    with pytest.raises(ContainerError, match="rank"):
        open_model(model_bytes(graph, tensors))
    tensors[1] = ("enc.w.scale", "F32", [2, 1], f32([1, 1]))
    with pytest.raises(ContainerError, match="broadcast"):
        open_model(model_bytes(graph, tensors))


def test_scale_key_may_not_be_an_initializers_tensor():
    graph = base_graph()
    graph["values"]["w"] = {"dtype": "f32", "shape": [3, 1]}
    graph["values"]["b"] = {"dtype": "f32", "shape": [3, 1]}
    graph["initializers"]["w"]["storage"] = {"dtype": "i8", "scale": "enc.b"}
    tensors = [("enc.b", "F32", [3, 1], f32([1, 2, 3])), ("enc.w", "I8", [3, 1], bytes(3))]
    with pytest.raises(ContainerError, match="collides"):
        open_model(model_bytes(graph, tensors))


def test_i4_storage_takes_a_group_shaped_scale():
    graph, tensors = i4_model()
    model = open_model(model_bytes(graph, tensors))
    assert model.initializers["w"].storage.group_size == 32
    assert model.file.tensors["enc.w"].byte_length == 128
    assert model.file.tensors["enc.w.scale"].shape == (4, 2)


@pytest.mark.parametrize("scale, fragment", [
    (("enc.w.scale", "F32", [8], f32([1] * 8)), "rank"),
    (("enc.w.scale", "F32", [4, 1], f32([1] * 4)), "group shape"),
    (("enc.w.scale", "F16", [4, 2], bytes(16)), "F32 needed"),
])
def test_i4_scale_that_is_not_group_shaped_is_rejected(scale, fragment):
    graph, tensors = i4_model(scale=scale)
    with pytest.raises(ContainerError, match=fragment):
        open_model(model_bytes(graph, tensors))


def test_rank3_i4_weight_takes_a_rank2_group_scale():
    def conv(scale):
        graph = base_graph()
        graph["values"]["w"] = {"dtype": "f32", "shape": [4, 8, 2]}
        graph["initializers"]["w"]["storage"] = {"dtype": "i4", "scale": "enc.w.scale",
                                                 "group_size": 16}
        return model_bytes(graph, [("enc.w", "I4", [4, 8, 2], bytes(32)), scale,
                                   BASE_TENSORS[1]])
    model = open_model(conv(("enc.w.scale", "F32", [4, 1], f32([1] * 4))))
    assert model.file.tensors["enc.w.scale"].shape == (4, 1)
    with pytest.raises(ContainerError, match="rank"):
        open_model(conv(("enc.w.scale", "F32", [4, 8, 1], f32([1] * 32))))
    with pytest.raises(ContainerError, match="group shape"):
        open_model(conv(("enc.w.scale", "F32", [4, 2], f32([1] * 8))))


# storage declaration rules: packages/runtime/src/format/ir.ts:268-305,620-650
@pytest.mark.parametrize("storage, fragment", [
    ({"dtype": "i4", "scale": "enc.w.scale"}, "needs group_size"),
    ({"dtype": "i4", "group_size": 32}, "needs scale"),
    ({"dtype": "i8"}, "needs scale"),
    ({"dtype": "f32", "scale": "enc.w.scale"}, "cannot carry"),
    ({"dtype": "f16", "group_size": 32}, "cannot carry"),
    ({"dtype": "i4", "scale": "enc.w.scale", "group_size": 8}, "power of two >= 16"),
    ({"dtype": "i4", "scale": "enc.w.scale", "group_size": 48}, "power of two >= 16"),
    ({"dtype": "i4", "scale": "enc.w.scale", "group_size": 32.0}, "positive integer"),
    ({"dtype": "i4", "scale": "enc.w.scale", "group_size": 0}, "positive integer"),
    ({"dtype": "i4", "scale": "", "group_size": 32}, "non-empty string"),
    ({"dtype": "i4", "scale": "enc.w.scale", "group_size": 128}, "not a multiple of group_size"),
    ({"dtype": "q4", "scale": "enc.w.scale"}, "unknown storage dtype"),
    ({"dtype": "i4", "scale": "enc.w.scale", "group_size": 32, "zero": 1}, "keys"),
])
def test_storage_declaration_rules(storage, fragment):
    graph, tensors = i4_model()
    graph["initializers"]["w"]["storage"] = storage
    with pytest.raises(IrError, match=fragment):
        open_model(model_bytes(graph, tensors))


def test_graph_version_and_format_are_checked():
    graph = base_graph()
    graph["version"] = 2
    with pytest.raises(IrError, match="version"):
        open_model(model_bytes(graph))
    graph = base_graph()
    graph["format"] = "onnx"
    with pytest.raises(IrError, match="karume-ir"):
        open_model(model_bytes(graph))
    with pytest.raises(IrError, match="cannot be parsed|non-finite"):
        open_model(build_safetensors(BASE_TENSORS, {"karume_ir": '{"version": NaN}'}))


def test_every_golden_model_file_opens():
    paths = sorted(glob.glob(os.path.join(helpers.GOLDEN, "*", "model.safetensors")))
    assert len(paths) >= 4
    for path in paths:
        with open(path, "rb") as handle:
            model = open_model(handle.read())
        assert set(model.initializers) <= set(model.graph["values"])
        assert i4_resident_initializers(model) == set()


def test_reference_i8_fixture_scales_are_matched():
    # data file of packages/runtime/tests/fixtures/golden/i8_weights: five I8 weights of rank
    # 2, 3 and 4, each with a keepdim F32 scale beside it
    with open(os.path.join(helpers.GOLDEN, "i8_weights", "model.safetensors"), "rb") as handle:
        blob = handle.read()
    model = open_model(blob)
    quantised = {n: i for n, i in model.initializers.items() if i.storage.dtype == "i8"}
    assert len(quantised) == 5
    for init in quantised.values():
        assert init.storage.scale == "karume.scale." + init.tensor
        scale = model.file.tensors[init.storage.scale]
        assert len(scale.shape) == len(init.shape)
    assert model.file.tensors["karume.scale.up.weight"].shape == (1, 2, 1)
    # dropping one scale tensor from the same file is caught
    file = model.file
    kept = [(n, v.dtype, v.shape, bytes(tensor_bytes(file, v))) for n, v in file.tensors.items()
            if n != "karume.scale.dense.weight"]
    kept.sort(key=lambda t: {"F32": 0, "I8": 1}[t[1]])
    with pytest.raises(ContainerError, match="scale tensor 'karume.scale.dense.weight'"):
        open_model(build_safetensors(kept, dict(file.metadata)))


# ---- residency rule: packages/runtime/src/runtime/plan.ts:366-431 -----------------------------

def resident(nodes, outputs=("y",), extra_inits=()):
    graph, tensors = i4_model()
    graph["nodes"] = nodes
    graph["outputs"] = list(outputs)
    return i4_resident_initializers(open_model(model_bytes(graph, tensors)))


def test_weight_slot_uses_keep_int4_packed():
    lin = {"op": "linear", "ins": ["x", "w", "b"], "outs": ["y"], "attrs": {}}
    emb = {"op": "embedding", "ins": ["w", "ids"], "outs": ["e"], "attrs": {"padding_idx": -1}}
    assert resident([lin]) == {"w"}
    assert resident([emb, lin]) == {"w"}          # tied table: both uses are weight slots
    conv = {"op": "conv1d", "ins": ["x", "w", "b"], "outs": ["y"],
            "attrs": {"stride": 1, "padding": 0, "dilation": 1, "groups": 1}}
    assert resident([conv]) == {"w"}


def test_other_uses_expand_int4_at_load():
    lin = {"op": "linear", "ins": ["x", "w", "b"], "outs": ["y"], "attrs": {}}
    assert resident([lin, {"op": "add", "ins": ["y", "w"], "outs": ["z"], "attrs": {}}]) == set()
    assert resident([{"op": "linear", "ins": ["w", "x"], "outs": ["y"], "attrs": {}}]) == set()
    assert resident([lin], outputs=("y", "w")) == set()
    assert resident([]) == set()
    grouped = {"op": "conv1d", "ins": ["x", "w", "b"], "outs": ["y"],
               "attrs": {"stride": 1, "padding": 0, "dilation": 1, "groups": 2}}
    assert resident([grouped]) == set()
    assert resident([lin, grouped]) == set()
    conv2d = {"op": "conv2d", "ins": ["x", "w", "b"], "outs": ["y"],
              "attrs": {"stride": [1, 1], "padding": [0, 0], "dilation": [1, 1], "groups": 1}}
    assert resident([conv2d]) == set()
    with pytest.raises(IrError, match="groups"):
        resident([{"op": "conv1d", "ins": ["x", "w", "b"], "outs": ["y"], "attrs": {}}])


# ---- packed payload hand-over ------------------------------------------------------------------

def test_packed_int4_views_decode_to_the_quantised_weight():
    rng = np.random.default_rng(5)
    codes = rng.integers(-8, 8, size=(4, 64))
    scales = rng.uniform(0.01, 0.2, size=(4, 2)).astype(np.float32)
    graph, tensors = i4_model()
    tensors[0] = ("enc.w", "I4", [4, 64], pack_int4(codes).tobytes())
    tensors[1] = ("enc.w.scale", "F32", [4, 2], scales.tobytes())
    model = open_model(model_bytes(graph, tensors))
    got = packed_int4(model, "w")
    assert got.shape == (4, 64) and got.group_size == 32
    assert got.packed.dtype == np.uint8 and got.packed.size == 128
    np.testing.assert_array_equal(got.scales, scales)
    dense = oracle.decode_i4(got.packed.tobytes(), [4, 64], got.scales.reshape(-1), [4, 2], 32)
    want = codes.astype(np.float32) * np.repeat(scales, 32, axis=1)
    np.testing.assert_array_equal(np.asarray(dense, dtype=np.float32).reshape(4, 64), want)
    with pytest.raises(ContainerError, match="not i4"):
        packed_int4(model, "b")
    with pytest.raises(ContainerError, match="no initializer"):
        packed_int4(model, "nope")
