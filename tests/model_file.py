"""Writes a decoder's weights as a Karume model file (safetensors + `karume_ir` graph) the way
the decode export recipe lays the graph out (tools/export-recipes/minicpm5/export_decode.py:
14-35; node vocabulary docs/ir-v1.md:277-520): token-only exit, RoPE as the exported 7-node
half-split chain over cos / sin rows looked up by position, states-form attention followed by
both appends.  Layers may differ the way a Gemma-4-style decoder's do
(tools/export-recipes/gemma4/export_decode.py:59-82,510-527): a `window` attr on the attention
and both appends of a sliding layer, a head dim (and RoPE tables) per layer kind, and KV-sharing
layers that read an earlier layer's roped k / v rows and slots and append nothing — the owner's
appends then follow its last reader in node order (docs/ir-v1.md:345-348).
Test-side only: the product reads such files, it does not write them."""
from __future__ import annotations

import json
from typing import Callable, Dict, List, Optional

import numpy as np

from karume_amd.decoder import DecoderWeights
from karume_amd.format_model import IR_METADATA_KEY, build_safetensors


def decoder_graph(weights: DecoderWeights, edit: Optional[Callable[[dict], None]] = None):
    """(graph dict, tensors list) for `weights`; `edit(graph)` may damage the graph first."""
    c = weights.config
    d, H, Hkv, V = c.d_model, c.heads, c.kv_heads, c.vocab
    nodes: List[dict] = []
    values: Dict[str, dict] = {}
    inits: Dict[str, dict] = {}
    tensors = []   # (key, dtype, shape, bytes)

    def value(name, shape, dtype="f32"):
        values[name] = {"dtype": dtype, "shape": list(shape)}
        return name

    def node(op, ins, outs, attrs=None, states=None):
        entry = {"op": op, "ins": list(ins), "outs": list(outs), "attrs": attrs or {}}
        if states is not None:
            entry["states"] = states
        nodes.append(entry)

    def f32_init(name, array):
        array = np.ascontiguousarray(array, dtype="<f4")
        inits[name] = {"tensor": name, "storage": {"dtype": "f32"}}
        value(name, array.shape)
        tensors.append((name, "F32", array.shape, array.tobytes()))
        return name

    def i4_init(name, lin):
        scale_key = f"karume.scale.{name}"
        inits[name] = {"tensor": name, "storage": {"dtype": "i4", "scale": scale_key,
                                                   "group_size": c.group_size}}
        value(name, (lin.n, lin.k))
        tensors.append((name, "I4", (lin.n, lin.k), np.ascontiguousarray(lin.packed).tobytes()))
        scales = np.ascontiguousarray(lin.scales, dtype="<f4")
        tensors.append((scale_key, "F32", scales.shape, scales.tobytes()))
        f32_init(f"{name}.bias", np.zeros(lin.n, dtype=np.float32))
        return name

    def linear(x, name, lin, out, lead):
        i4_init(name, lin)
        node("linear", [x, name, f"{name}.bias"], [value(out, (*lead, lin.n))])
        return out

    def rope(x, heads, tag, D):
        half = D // 2
        cos, sin = f"cos{D}", f"sin{D}"
        shape_full, shape_half = (1, heads, "M", D), (1, heads, "M", half)
        a, b, nb, rot, direct, cross, out = (f"{tag}.{s}" for s in
                                             ("lo", "hi", "neg", "rot", "xc", "rs", "rope"))
        node("slice", [x], [value(a, shape_half)], {"dim": 3, "start": 0, "end": half})
        node("slice", [x], [value(b, shape_half)], {"dim": 3, "start": half, "end": D})
        node("neg", [b], [value(nb, shape_half)])
        node("cat", [nb, a], [value(rot, shape_full)], {"dim": 3})
        node("mul", [x, cos], [value(direct, shape_full)])
        node("mul", [rot, sin], [value(cross, shape_full)])
        node("add", [direct, cross], [value(out, shape_full)])
        return out

    inputs = [{"name": "input_ids", "dtype": "i32", "shape": [1, "M"]},
              {"name": "position_ids", "dtype": "i32", "shape": [1, "M"]},
              {"name": "last_row", "dtype": "i32", "shape": [1]}]
    embedding = np.ascontiguousarray(weights.embedding, dtype="<f2")
    inits["embed"] = {"tensor": "embed", "storage": {"dtype": "f16"}}
    value("embed", (V, d))
    node("embedding", ["embed", "input_ids"], [value("h.in", (1, "M", d))], {"padding_idx": None})
    for D in c.head_dims:
        for table, array in zip(("cos", "sin"), weights.rope_of(D)):
            f32_init(f"rope.{table}{D}", array)
            node("embedding", [f"rope.{table}{D}", "position_ids"],
                 [value(f"{table}{D}.rows", (1, "M", D))], {"padding_idx": None})
            node("reshape", [f"{table}{D}.rows"], [value(f"{table}{D}", (1, 1, "M", D))])
    states = {}
    h = "h.in"
    step_kv = {}      # owner layer -> (roped k value, v value) of this step
    for li, lw in enumerate(weights.layers):
        p = f"l{li}"
        D, owner, window = c.depth_of(li), c.owner_of(li), c.window_of(li)
        window_attr = {"window": window} if window else {}
        f32_init(f"{p}.attn_norm", lw["attn_norm"])
        node("rms_norm", [h, f"{p}.attn_norm"], [value(f"{p}.xn", (1, "M", d))], {"eps": c.rms_eps})
        heads_of = {"q": H, "k": Hkv, "v": Hkv}
        head_major = {}
        for slot in ("q", "k", "v") if owner == li else ("q",):
            flat = linear(f"{p}.xn", f"{p}.{slot}_proj", lw[slot], f"{p}.{slot}.flat", (1, "M"))
            node("reshape", [flat], [value(f"{p}.{slot}.rows", (1, "M", heads_of[slot], D))])
            node("permute", [f"{p}.{slot}.rows"],
                 [value(f"{p}.{slot}", (1, heads_of[slot], "M", D))], {"dims": [0, 2, 1, 3]})
            head_major[slot] = f"{p}.{slot}"
        q_rot = rope(head_major["q"], H, f"{p}.q", D)
        if owner == li:
            states[f"{p}.k"] = {"dtype": "f32", "shape": [1, Hkv, "C", D]}
            states[f"{p}.v"] = {"dtype": "f32", "shape": [1, Hkv, "C", D]}
            step_kv[li] = (rope(head_major["k"], Hkv, f"{p}.k", D), head_major["v"])
        k_rot, v_rows = step_kv[owner]
        node("attention", [q_rot, k_rot, v_rows], [value(f"{p}.att", (1, H, "M", D))],
             {"scale": float(np.float32(c.half_scale_of(li))), **window_attr},
             {"k": f"l{owner}.k", "v": f"l{owner}.v"})
        if c.readers_of(owner)[-1] == li:   # the appends follow the slot's last reader
            node("state_append", [k_rot], [], dict(window_attr), {"slot": f"l{owner}.k"})
            node("state_append", [v_rows], [], dict(window_attr), {"slot": f"l{owner}.v"})
        node("permute", [f"{p}.att"], [value(f"{p}.att.rows", (1, "M", H, D))], {"dims": [0, 2, 1, 3]})
        node("reshape", [f"{p}.att.rows"], [value(f"{p}.att.flat", (1, "M", H * D))])
        o = linear(f"{p}.att.flat", f"{p}.o_proj", lw["o"], f"{p}.o", (1, "M"))
        node("add", [h, o], [value(f"{p}.h1", (1, "M", d))])
        f32_init(f"{p}.ffn_norm", lw["ffn_norm"])
        node("rms_norm", [f"{p}.h1", f"{p}.ffn_norm"], [value(f"{p}.xn2", (1, "M", d))],
             {"eps": c.rms_eps})
        gate = linear(f"{p}.xn2", f"{p}.gate_proj", lw["gate"], f"{p}.gate", (1, "M"))
        node("sigmoid", [gate], [value(f"{p}.gate.sig", (1, "M", c.ffn))])
        node("mul", [gate, f"{p}.gate.sig"], [value(f"{p}.gate.silu", (1, "M", c.ffn))])
        up = linear(f"{p}.xn2", f"{p}.up_proj", lw["up"], f"{p}.up", (1, "M"))
        node("mul", [f"{p}.gate.silu", up], [value(f"{p}.act", (1, "M", c.ffn))])
        down = linear(f"{p}.act", f"{p}.down_proj", lw["down"], f"{p}.down", (1, "M"))
        node("add", [f"{p}.h1", down], [value(f"{p}.h2", (1, "M", d))])
        h = f"{p}.h2"
    f32_init("final_norm", weights.final_norm)
    node("rms_norm", [h, "final_norm"], [value("h.norm", (1, "M", d))], {"eps": c.rms_eps})
    node("reshape", ["h.norm"], [value("h.rows", ("M", d))])
    node("embedding", ["h.rows", "last_row"], [value("h.last", (1, d))], {"padding_idx": None})
    node("reshape", ["h.last"], [value("h.last.row", (1, 1, d))])
    linear("h.last.row", "lm_head", weights.lm_head, "logits", (1, 1))
    node("argmax", ["logits"], [value("token", (1, 1, 1), "i32")])
    tensors.append(("embed", "F16", embedding.shape, embedding.tobytes()))  # 2-byte aligned: last
    graph = {"format": "karume-ir", "version": 1,
             "requires": {"ops": sorted({n["op"] for n in nodes})}, "symbols": ["M", "C"],
             "inputs": inputs, "outputs": ["logits", "token"], "initializers": inits,
             "values": values, "states": states, "nodes": nodes}
    if edit is not None:
        edit(graph)
    return graph, tensors


def decoder_model_file(weights: DecoderWeights, edit=None, edit_tensors=None) -> bytes:
    graph, tensors = decoder_graph(weights, edit)
    if edit_tensors is not None:
        tensors = edit_tensors(tensors)
    return build_safetensors(tensors, {IR_METADATA_KEY: json.dumps(graph)})
