"""A model file's graph -> the weights of a Llama-style int4 decoder session.

The reference turns a `karume_ir` graph into a plan generically (container
packages/runtime/src/format/container.ts:343-384,468-506, int4 residency
packages/runtime/src/runtime/plan.ts:366-431) and runs whatever nodes it holds.  This backend
runs one graph shape — the states-form decode graph of a Llama / MiniCPM5-style decoder in the
node order the export recipe emits (tools/export-recipes/minicpm5/export_decode.py:14-35):

    embedding(ids) -> per layer [ rms_norm -> q/k/v linear -> reshape/permute -> rope(q), rope(k)
                                  -> attention(states k, v) -> state_append(k), state_append(v)
                                  -> permute/reshape -> o linear -> add
                                  -> rms_norm -> gate/up linear -> silu(gate) * up -> down linear -> add ]
                   -> rms_norm -> lm_head linear -> argmax

Layers may differ the way a Gemma-4-style decoder's do (tools/export-recipes/gemma4/
export_decode.py:59-82,510-527): a `window` attr on the attention and the appends of a sliding
layer, a head dim (with RoPE tables of its own) per layer kind, and KV-sharing layers, whose
attention reads the roped k / v rows and the state slots of an earlier layer and which append
nothing (two readers, one append; the owner's appends must follow its last reader,
docs/ir-v1.md:345-348).  What else such models add around the attention (per-layer embedding
tables, q / k norms, GELU, logit soft-capping) is not this graph shape and is rejected.

So loading is recognition, not compilation: every attention node is traced back to the
linears that feed it and forward to the linears that consume it, and anything that does not fit
the shape above is rejected by name (nothing is approximated or skipped silently).  RoPE is the
exported 7-node half-split chain (slice, slice, neg, cat, mul, mul, add in either of the two
orders packages/runtime/src/runtime/fusion.ts:633-760 accepts) over cos / sin rows looked up
from two tables by position (`embedding(table, position_ids)`).
"""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np

from .decoder import DecoderWeights, Int4Linear, LlamaConfig
from .format_model import (ContainerError, IrError, KarumeModel, i4_resident_initializers,
                           packed_int4, tensor_bytes)

_LAYOUT_OPS = ("reshape", "permute", "expand")


class GraphShapeError(IrError):
    """The graph is valid IR but not the decoder shape this backend runs."""


class _Graph:
    def __init__(self, model: KarumeModel):
        graph = model.graph
        self.model = model
        self.nodes: List[dict] = graph.get("nodes", [])
        self.values: Dict[str, dict] = graph.get("values", {})
        self.inputs = {item["name"]: item for item in graph.get("inputs", [])}
        self.producer: Dict[str, int] = {}
        self.users: Dict[str, List[int]] = {}
        for index, node in enumerate(self.nodes):
            for name in node.get("outs", []):
                self.producer[name] = index
            for name in node.get("ins", []):
                self.users.setdefault(name, []).append(index)

    def shape(self, name: str) -> list:
        if name in self.inputs:
            return list(self.inputs[name]["shape"])
        info = self.values.get(name)
        if info is None:
            raise GraphShapeError(f"value '{name}' has no declared shape")
        return list(info["shape"])

    def node_of(self, name: str) -> Optional[dict]:
        index = self.producer.get(name)
        return None if index is None else self.nodes[index]

    def through_layout(self, name: str) -> str:
        """The value behind any run of reshape / permute / expand nodes."""
        while True:
            node = self.node_of(name)
            if node is None or node["op"] not in _LAYOUT_OPS:
                return name
            name = node["ins"][0]

    def sole_user(self, name: str, what: str) -> Tuple[int, dict]:
        users = self.users.get(name, [])
        if len(users) != 1:
            raise GraphShapeError(f"{what} '{name}' has {len(users)} readers (1 expected)")
        return users[0], self.nodes[users[0]]

    def forward_through_layout(self, name: str, what: str) -> Tuple[str, dict]:
        """Follow a value through layout nodes to its first non-layout reader."""
        while True:
            _, node = self.sole_user(name, what)
            if node["op"] not in _LAYOUT_OPS:
                return name, node
            name = node["outs"][0]


def _rope_source(g: _Graph, name: str, what: str) -> Tuple[str, Optional[Tuple[str, str]]]:
    """If `name` is the `add` that ends a half-split RoPE chain, return (x, (cos value, sin
    value)); otherwise (name, None).  The chain is checked edge by edge."""
    add = g.node_of(name)
    if add is None or add["op"] != "add":
        return name, None
    direct, cross = g.node_of(add["ins"][0]), g.node_of(add["ins"][1])
    if direct is None or cross is None or direct["op"] != "mul" or cross["op"] != "mul":
        raise GraphShapeError(f"{what}: '{name}' is an add that is not x*cos + rotate_half(x)*sin")
    x = direct["ins"][0]
    cat = g.node_of(cross["ins"][0])
    if cat is None or cat["op"] != "cat" or cat.get("attrs", {}).get("dim") != 3:
        raise GraphShapeError(f"{what}: the RoPE cross term does not read cat(dim=3)")
    neg, first = g.node_of(cat["ins"][0]), g.node_of(cat["ins"][1])
    second = g.node_of(neg["ins"][0]) if neg is not None and neg["op"] == "neg" else None
    if first is None or second is None or first["op"] != "slice" or second["op"] != "slice":
        raise GraphShapeError(f"{what}: the RoPE chain is not cat(neg(slice), slice)")
    depth = g.shape(x)[-1]
    if not isinstance(depth, int) or depth < 2 or depth % 2:
        raise GraphShapeError(f"{what}: head dim {depth!r} is not a positive even number")
    half = depth // 2
    want_first = {"dim": 3, "start": 0, "end": half}
    want_second = {"dim": 3, "start": half, "end": depth}
    if first["ins"][0] != x or second["ins"][0] != x or first.get("attrs") != want_first or \
            second.get("attrs") != want_second:
        raise GraphShapeError(f"{what}: the RoPE slices are not [0, D/2) and [D/2, D) of one value")
    return x, (direct["ins"][1], cross["ins"][1])


def _table_of(g: _Graph, value: str, positions: str, what: str) -> str:
    """Initializer behind cos / sin rows: embedding(table, position_ids) behind layout nodes."""
    node = g.node_of(g.through_layout(value))
    if node is None or node["op"] != "embedding" or node["ins"][1] != positions:
        raise GraphShapeError(f"{what}: '{value}' is not a table looked up by '{positions}'")
    table = node["ins"][0]
    if table not in g.model.initializers:
        raise GraphShapeError(f"{what}: table '{table}' is not an initializer")
    return table


def _f32_initializer(g: _Graph, name: str, what: str) -> np.ndarray:
    init = g.model.initializers.get(name)
    if init is None:
        raise GraphShapeError(f"{what}: '{name}' is not an initializer")
    view = g.model.file.tensors[init.tensor]
    raw = tensor_bytes(g.model.file, view)
    if init.storage.dtype == "f32":
        data = np.frombuffer(raw, dtype="<f4")
    elif init.storage.dtype == "f16":
        data = np.frombuffer(raw, dtype="<f2")
    else:
        raise GraphShapeError(f"{what}: '{name}' is stored as {init.storage.dtype}; this session "
                              "takes f32 or f16 storage here")
    return data.reshape(init.shape)


def _linear(g: _Graph, node: dict, resident: set, what: str) -> Tuple[Int4Linear, int]:
    """The int4 weight of a `linear` node (bias must be all zeros: the session binds none)."""
    if node["op"] != "linear" or len(node["ins"]) != 3:
        raise GraphShapeError(f"{what}: expected a linear node, found '{node['op']}'")
    weight, bias = node["ins"][1], node["ins"][2]
    if weight not in resident:
        raise GraphShapeError(f"{what}: weight '{weight}' is not an int4-resident initializer "
                              "(this session runs int4 linears only)")
    w = packed_int4(g.model, weight)
    if len(w.shape) != 2:
        raise GraphShapeError(f"{what}: weight '{weight}' has rank {len(w.shape)} (2 expected)")
    if np.any(_f32_initializer(g, bias, what)):
        raise GraphShapeError(f"{what}: bias '{bias}' is not all zeros; the decoder session "
                              "binds no bias")
    n, k = w.shape
    return Int4Linear(n, k, w.packed.reshape(n, k // 2), w.scales), w.group_size


def decoder_weights_from_model(model: KarumeModel) -> DecoderWeights:
    """DecoderWeights (host views into the file's buffer where the layout allows) for a model
    file whose graph is the Llama-style states-form decode graph; GraphShapeError otherwise."""
    g = _Graph(model)
    resident = i4_resident_initializers(model)
    int_inputs = [item["name"] for item in model.graph.get("inputs", []) if item["dtype"] == "i32"]
    attentions = [node for node in g.nodes if node["op"] == "attention"]
    if not attentions:
        raise GraphShapeError("the graph holds no attention node")

    # token embedding: the embedding whose index is a graph input and whose table is [V, d]
    token_nodes = [n for n in g.nodes if n["op"] == "embedding" and n["ins"][1] in int_inputs
                   and len(g.shape(n["outs"][0])) == 3 and
                   g.users.get(n["outs"][0], []) and
                   any(g.nodes[u]["op"] in ("rms_norm", "add") for u in g.users[n["outs"][0]])]
    if len(token_nodes) != 1:
        raise GraphShapeError(f"{len(token_nodes)} token embedding nodes (1 expected)")
    ids_input = token_nodes[0]["ins"][1]
    embedding = _f32_initializer(g, token_nodes[0]["ins"][0], "token embedding")
    vocab, d_model = embedding.shape
    others = [name for name in int_inputs if name != ids_input]
    if not others:
        raise GraphShapeError("the graph has no position input")

    group_sizes, eps_values = set(), set()
    layers: List[Dict[str, object]] = []
    tables: Dict[int, Tuple[str, str]] = {}     # head dim -> (cos table, sin table)
    positions = None
    heads = kv_heads = None
    depths: List[int] = []
    windows: List[int] = []
    owners: List[int] = []
    kv_linear_owner: Dict[int, int] = {}        # index of a k / v linear node -> its layer
    att_index = {id(node): index for index, node in enumerate(g.nodes)}
    for li, att in enumerate(attentions):
        what = f"layer {li}"
        states = att.get("states")
        if not isinstance(states, dict) or set(states) != {"k", "v"}:
            raise GraphShapeError(f"{what}: the attention node is not in states form")
        window = att.get("attrs", {}).get("window", 0)
        if not isinstance(window, int) or isinstance(window, bool) or window < 0:
            raise GraphShapeError(f"{what}: window {window!r} is not a positive integer")
        q_shape, k_shape = g.shape(att["ins"][0]), g.shape(att["ins"][1])
        dims = (q_shape[1], k_shape[1])
        depth = q_shape[3]
        if heads is None:
            heads, kv_heads = dims
        elif dims != (heads, kv_heads):
            raise GraphShapeError(f"{what}: heads / kv heads {dims} differ from layer 0")
        if not isinstance(depth, int) or k_shape[3] != depth or g.shape(att["ins"][2])[3] != depth:
            raise GraphShapeError(f"{what}: q, k and v do not share one head dim")
        want_scale = float(np.float32(np.sqrt(1.0 / np.sqrt(float(depth)))))
        scale = float(att["attrs"]["scale"])
        if abs(scale - want_scale) > 1e-6 * want_scale:
            raise GraphShapeError(f"{what}: attention scale {scale} is not sqrt(1/sqrt({depth})) "
                                  f"= {want_scale}")

        entry: Dict[str, object] = {}
        norm_inputs = set()
        kv_nodes = []
        for slot, name in zip(("q", "k", "v"), att["ins"]):
            source, found = _rope_source(g, g.through_layout(name), f"{what}.{slot}")
            if (found is not None) != (slot != "v"):
                raise GraphShapeError(f"{what}.{slot}: RoPE is expected on q and k and not on v")
            if found is not None:
                for other in others:
                    try:
                        pair = (_table_of(g, found[0], other, what), _table_of(g, found[1], other, what))
                    except GraphShapeError:
                        continue
                    if positions is None:
                        positions = other
                    if other != positions or tables.setdefault(depth, pair) != pair:
                        raise GraphShapeError(f"{what}.{slot}: a second pair of RoPE tables for "
                                              f"head dim {depth}")
                    break
                else:
                    raise GraphShapeError(f"{what}.{slot}: cos / sin are not looked up by position")
            node_index = g.producer.get(g.through_layout(source))
            if node_index is None:
                raise GraphShapeError(f"{what}.{slot}: no linear node behind '{source}'")
            node = g.nodes[node_index]
            if slot != "q":
                kv_nodes.append(node_index)
                if node_index in kv_linear_owner:
                    continue          # the k / v rows of an earlier layer (checked below)
            entry[slot], group = _linear(g, node, resident, f"{what}.{slot}")
            group_sizes.add(group)
            norm_inputs.add(node["ins"][0])
        shared_from = {kv_linear_owner.get(index) for index in kv_nodes}
        if shared_from == {None}:
            owner = li
            for index in kv_nodes:
                kv_linear_owner[index] = li
        elif len(shared_from) == 1:
            # a KV-sharing layer: k and v are the rows of ONE earlier layer, read from that
            # layer's slots under the same window
            owner = shared_from.pop()
            owner_att = attentions[owner]
            if owner_att["ins"][1] != att["ins"][1] or owner_att["ins"][2] != att["ins"][2] or \
                    owner_att["states"] != states:
                raise GraphShapeError(f"{what}: reads the k / v linears of layer {owner} but not "
                                      "its roped rows and state slots")
            if depths[owner] != depth or windows[owner] != window:
                raise GraphShapeError(f"{what}: shares the K / V of layer {owner} under another "
                                      "head dim or window")
        else:
            raise GraphShapeError(f"{what}: k and v come from different layers")
        depths.append(depth)
        windows.append(window)
        owners.append(owner)
        if len(norm_inputs) != 1:
            raise GraphShapeError(f"{what}: q, k and v do not read one normalised row")
        norm = g.node_of(next(iter(norm_inputs)))
        if norm is None or norm["op"] != "rms_norm":
            raise GraphShapeError(f"{what}: q / k / v do not read an rms_norm")
        entry["attn_norm"] = np.ascontiguousarray(_f32_initializer(g, norm["ins"][1], what),
                                                   dtype=np.float32)
        eps_values.add(float(norm["attrs"]["eps"]))

        # forward: attention -> o linear -> add -> rms_norm -> gate / up -> silu * up -> down -> add
        _, o_node = g.forward_through_layout(att["outs"][0], f"{what} attention output")
        entry["o"], group = _linear(g, o_node, resident, f"{what}.o")
        group_sizes.add(group)
        _, add1 = g.sole_user(o_node["outs"][0], f"{what} o output")
        if add1["op"] != "add":
            raise GraphShapeError(f"{what}: the o projection does not feed a residual add")
        ffn_norms = [g.nodes[u] for u in g.users.get(add1["outs"][0], [])
                     if g.nodes[u]["op"] == "rms_norm"]
        if len(ffn_norms) != 1:
            raise GraphShapeError(f"{what}: no rms_norm after the attention residual")
        entry["ffn_norm"] = np.ascontiguousarray(
            _f32_initializer(g, ffn_norms[0]["ins"][1], what), dtype=np.float32)
        eps_values.add(float(ffn_norms[0]["attrs"]["eps"]))
        branches = [g.nodes[u] for u in g.users.get(ffn_norms[0]["outs"][0], [])]
        if len(branches) != 2 or any(b["op"] != "linear" for b in branches):
            raise GraphShapeError(f"{what}: the FFN norm does not feed exactly gate and up")
        gate = up = None
        product = None
        for b in branches:
            out = b["outs"][0]
            ops = sorted(g.nodes[u]["op"] for u in g.users.get(out, []))
            if ops == ["mul", "sigmoid"]:       # silu(gate) = gate * sigmoid(gate)
                sig = next(g.nodes[u] for u in g.users[out] if g.nodes[u]["op"] == "sigmoid")
                silu = next(g.nodes[u] for u in g.users[out] if g.nodes[u]["op"] == "mul")
                if set(silu["ins"]) != {out, sig["outs"][0]}:
                    raise GraphShapeError(f"{what}: gate is not followed by gate * sigmoid(gate)")
                gate = b
                _, product = g.sole_user(silu["outs"][0], f"{what} silu output")
            elif ops == ["mul"]:
                up = b
            else:
                raise GraphShapeError(f"{what}: an FFN branch is read by {ops}")
        if gate is None or up is None or product is None or product["op"] != "mul" or \
                up["outs"][0] not in product["ins"]:
            raise GraphShapeError(f"{what}: the FFN is not silu(gate) * up")
        entry["gate"], g1 = _linear(g, gate, resident, f"{what}.gate")
        entry["up"], g2 = _linear(g, up, resident, f"{what}.up")
        _, down = g.sole_user(product["outs"][0], f"{what} FFN product")
        entry["down"], g3 = _linear(g, down, resident, f"{what}.down")
        group_sizes.update((g1, g2, g3))
        _, add2 = g.sole_user(down["outs"][0], f"{what} down output")
        if add2["op"] != "add" or add1["outs"][0] not in add2["ins"]:
            raise GraphShapeError(f"{what}: the down projection does not feed a residual add")
        layers.append(entry)

    # every owner's slots are appended once each, from its own roped k rows and v rows, under
    # the layer's window, after the last attention that reads them (docs/ir-v1.md:345-348)
    appends = {}
    for index, node in enumerate(g.nodes):
        if node["op"] == "state_append":
            slot = node["states"]["slot"]
            if slot in appends:
                raise GraphShapeError(f"state slot '{slot}' is appended twice")
            appends[slot] = (index, node)
    for li, att in enumerate(attentions):
        if owners[li] != li:
            continue
        readers = [index for index, other in enumerate(attentions) if owners[index] == li]
        last_reader = max(att_index[id(attentions[index])] for index in readers)
        for slot, source in ((att["states"]["k"], att["ins"][1]), (att["states"]["v"], att["ins"][2])):
            if slot not in appends:
                raise GraphShapeError(f"layer {li}: no state_append for slot '{slot}' (a layer "
                                      "that appends nothing must read another layer's k / v)")
            index, node = appends[slot]
            if node["ins"][0] != source:
                raise GraphShapeError(f"layer {li}: slot '{slot}' is appended from "
                                      f"'{node['ins'][0]}', not from the rows the attention reads")
            if node.get("attrs", {}).get("window", 0) != windows[li]:
                raise GraphShapeError(f"layer {li}: the append of '{slot}' declares another window "
                                      "than the attention")
            if index < last_reader:
                raise GraphShapeError(f"layer {li}: slot '{slot}' is appended before its last "
                                      "reader")

    # exit: argmax <- lm_head linear <- rms_norm
    argmaxes = [n for n in g.nodes if n["op"] == "argmax"]
    if len(argmaxes) != 1:
        raise GraphShapeError(f"{len(argmaxes)} argmax nodes (1 expected)")
    head = g.node_of(g.through_layout(argmaxes[0]["ins"][0]))
    if head is None:
        raise GraphShapeError("the argmax does not read a linear")
    lm_head, group = _linear(g, head, resident, "lm_head")
    group_sizes.add(group)
    final_source = g.through_layout(head["ins"][0])
    final = g.node_of(final_source)
    # the token-only exit selects the last valid row first: embedding(hidden rows, last_row)
    # (docs/decisions/0068-decode-exit-multi-output.md:148-160)
    while final is not None and final["op"] == "embedding" and \
            final["ins"][0] not in model.initializers:
        final = g.node_of(g.through_layout(final["ins"][0]))
    if final is None or final["op"] != "rms_norm":
        raise GraphShapeError("the lm_head does not read an rms_norm")
    eps_values.add(float(final["attrs"]["eps"]))

    if len(group_sizes) != 1 or len(eps_values) != 1:
        raise GraphShapeError(f"group sizes {sorted(group_sizes)} and eps {sorted(eps_values)} "
                              "must each be uniform")
    rope = {}
    for depth, (cos_table, sin_table) in tables.items():
        cos = np.ascontiguousarray(_f32_initializer(g, cos_table, "RoPE cos table"), dtype=np.float32)
        sin = np.ascontiguousarray(_f32_initializer(g, sin_table, "RoPE sin table"), dtype=np.float32)
        if cos.shape != sin.shape or cos.ndim != 2 or cos.shape[1] != depth:
            raise GraphShapeError(f"RoPE tables {cos.shape} / {sin.shape} are not "
                                  f"[positions, {depth}]")
        rope[depth] = (cos, sin)
    if len({cos.shape[0] for cos, _ in rope.values()}) != 1:
        raise GraphShapeError("the RoPE tables of the layer kinds differ in length")
    for li, entry in enumerate(layers):
        if entry["q"].n != heads * depths[li] or entry["q"].k != d_model or \
                (owners[li] == li and entry["k"].n != kv_heads * depths[li]):
            raise GraphShapeError(f"layer {li}: projection shapes disagree with heads x head dim "
                                  "/ d_model")
    uniform = len(set(depths)) == 1 and not any(windows) and owners == list(range(len(layers)))
    depth0 = depths[0]
    config = LlamaConfig(layers=len(layers), d_model=int(d_model), ffn=int(layers[0]["gate"].n),
                         heads=int(heads), kv_heads=int(kv_heads), head_dim=int(depth0),
                         vocab=int(vocab), group_size=int(next(iter(group_sizes))),
                         rms_eps=float(next(iter(eps_values))),
                         max_position=int(rope[depth0][0].shape[0]),
                         layer_windows=() if uniform else tuple(windows),
                         layer_head_dims=() if uniform else tuple(depths),
                         layer_kv_source=() if uniform else tuple(owners))
    if lm_head.n != vocab or lm_head.k != d_model:
        raise GraphShapeError("the lm_head shape disagrees with the embedding table")
    weights = DecoderWeights(config, np.ascontiguousarray(embedding, dtype=np.float16))
    if not np.array_equal(weights.embedding.astype(np.float32), embedding.astype(np.float32)):
        raise GraphShapeError("the token embedding table does not fit fp16 exactly; this session "
                              "keeps it in fp16")
    weights.layers = layers
    weights.final_norm = np.ascontiguousarray(_f32_initializer(g, final["ins"][1], "final norm"),
                                              dtype=np.float32)
    weights.lm_head = lm_head
    weights.rope_cos, weights.rope_sin = rope[depth0]
    weights.rope_by_depth = {depth: pair for depth, pair in rope.items() if depth != depth0}
    return weights


__all__ = ["GraphShapeError", "decoder_weights_from_model"]
