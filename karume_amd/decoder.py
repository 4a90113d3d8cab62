"""A Llama-style int4 decoder driven through the C ABI — the decode graph the reference exports
(tools/export-recipes/minicpm5/export_decode.py:14-35), op for op:

    embedding -> per layer [ rms_norm -> q/k/v linear -> rope(q, k) -> attention(states)
                             -> state_append(k), state_append(v) -> o linear -> add
                             -> rms_norm -> gate/up linear -> silu*mul -> down linear -> add ]
              -> rms_norm(last valid row) -> lm_head linear -> argmax

``run`` has the shape of the reference's ``Session.run`` for that graph (ids and positions of
the chunk in, argmax token of the last valid row out; the context's lengths advance on success
and the context is poisoned on failure).  ``decode_tokens`` replays one recorded decode step
with the lengths, the positions and the fed-back token all living on the device, so the greedy
loop needs no per-step read-back.

Every tensor operation is a call into libkarume_hip.so; this module only sequences them.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np

from .format_i4 import pack_int4
from .generation import GenerationContext
from .runtime import (COMPUTE_F16, COMPUTE_F32, F16, F32, DeviceBuffer, ExecutionError,
                      GpuContext, KarumeError)


@dataclass(frozen=True)
class LlamaConfig:
    layers: int = 22
    d_model: int = 2048
    ffn: int = 5632
    heads: int = 32
    kv_heads: int = 4
    head_dim: int = 64
    vocab: int = 32000
    group_size: int = 128
    rms_eps: float = 1e-5
    rope_base: float = 10000.0
    max_position: int = 512
    # Per-layer attention structure (empty = the same for every layer), as Gemma-4-style decoders
    # declare it (tools/export-recipes/gemma4/export_decode.py:59-82,510-527):
    #   layer_windows[l]   sliding window of layer l's state slots, 0 = full context
    #   layer_head_dims[l] head dim of layer l (sliding and full layers differ there)
    #   layer_kv_source[l] the layer whose K / V layer l attends over: l itself, or an earlier
    #                      layer for a KV-sharing layer (which has no k / v projection and
    #                      appends nothing: two readers, one append)
    layer_windows: tuple = ()
    layer_head_dims: tuple = ()
    layer_kv_source: tuple = ()

    def __post_init__(self):
        for name in ("layer_windows", "layer_head_dims", "layer_kv_source"):
            value = tuple(int(v) for v in getattr(self, name))
            if value and len(value) != self.layers:
                raise ValueError(f"{name} has {len(value)} entries for {self.layers} layers")
            object.__setattr__(self, name, value)
        for layer, source in enumerate(self.layer_kv_source):
            if not 0 <= source <= layer or self.layer_kv_source[source] != source:
                raise ValueError(f"layer {layer} takes its K / V from layer {source}, which is "
                                 "not an earlier layer that owns its own")
            if source != layer and (self.depth_of(source) != self.depth_of(layer)
                                    or self.window_of(source) != self.window_of(layer)):
                raise ValueError(f"layer {layer} shares the K / V of layer {source} but declares "
                                 "another head dim or window")

    @property
    def half_scale(self) -> float:
        return float(np.float32(np.sqrt(1.0 / np.sqrt(float(self.head_dim)))))

    def window_of(self, layer: int) -> int:
        return self.layer_windows[layer] if self.layer_windows else 0

    def depth_of(self, layer: int) -> int:
        return self.layer_head_dims[layer] if self.layer_head_dims else self.head_dim

    def owner_of(self, layer: int) -> int:
        return self.layer_kv_source[layer] if self.layer_kv_source else layer

    def half_scale_of(self, layer: int) -> float:
        return float(np.float32(np.sqrt(1.0 / np.sqrt(float(self.depth_of(layer))))))

    @property
    def head_dims(self) -> tuple:
        """The distinct head dims, ascending (one pair of RoPE tables each)."""
        return tuple(sorted({self.depth_of(l) for l in range(self.layers)}))

    def readers_of(self, layer: int) -> list:
        """Layers that attend over the K / V of `layer` (itself first)."""
        return [l for l in range(self.layers) if self.owner_of(l) == layer]


@dataclass
class Int4Linear:
    """Host copy of one quantised linear: packed [N, K/2] bytes and [N, K/g] scales."""
    n: int
    k: int
    packed: np.ndarray
    scales: np.ndarray  # float16


@dataclass
class DecoderWeights:
    config: LlamaConfig
    embedding: np.ndarray                      # [vocab, d_model] float16
    layers: List[Dict[str, object]] = field(default_factory=list)
    final_norm: np.ndarray = None              # [d_model] float32
    lm_head: Int4Linear = None
    rope_cos: np.ndarray = None                # [max_position, head_dim] float32
    rope_sin: np.ndarray = None
    # layers of another head dim look their rotation up in tables of their own:
    # head dim -> (cos, sin), each [max_position, head dim]; head_dim itself stays above
    rope_by_depth: Dict[int, tuple] = field(default_factory=dict)

    def rope_of(self, depth: int):
        if depth == self.config.head_dim:
            return self.rope_cos, self.rope_sin
        return self.rope_by_depth[depth]

    @staticmethod
    def from_model(model) -> "DecoderWeights":
        """Weights of a model file (karume_amd.open_model) whose graph is the Llama-style
        states-form decode graph; see karume_amd.decoder_loader."""
        from .decoder_loader import decoder_weights_from_model

        return decoder_weights_from_model(model)


def rope_tables(config: LlamaConfig, depth: Optional[int] = None):
    """cos / sin rows for positions 0..max_position-1, half-split convention (the two halves of
    a row repeat the same angles), computed in float64 and stored as float32."""
    half = (config.head_dim if depth is None else depth) // 2
    inv_freq = 1.0 / (config.rope_base ** (np.arange(half, dtype=np.float64) / half))
    angles = np.arange(config.max_position, dtype=np.float64)[:, None] * inv_freq[None, :]
    angles = np.concatenate([angles, angles], axis=1)
    return np.cos(angles).astype(np.float32), np.sin(angles).astype(np.float32)


def random_weights(config: LlamaConfig, seed: int = 0) -> DecoderWeights:
    """Random-init weights of the benchmark's shape: int4 codes uniform in [-8, 7], fp16 scales
    |N(0, 0.02)|, fp16 embeddings N(0, 0.02), norm weights 1."""
    rng = np.random.default_rng(seed)

    def lin(n: int, k: int) -> Int4Linear:
        packed = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
        scales = np.maximum(np.abs(rng.normal(0, 0.02, size=(n, k // config.group_size)))
                            .astype(np.float16), np.float16(6.104e-05))
        return Int4Linear(n, k, packed, scales)

    d = config.d_model
    w = DecoderWeights(config, rng.normal(0, 0.02, size=(config.vocab, d)).astype(np.float16))
    for layer in range(config.layers):
        depth = config.depth_of(layer)
        kv = config.kv_heads * depth
        entry = {
            "attn_norm": np.ones(d, dtype=np.float32), "ffn_norm": np.ones(d, dtype=np.float32),
            "q": lin(config.heads * depth, d), "k": lin(kv, d), "v": lin(kv, d),
            "o": lin(d, config.heads * depth),
            "gate": lin(config.ffn, d), "up": lin(config.ffn, d), "down": lin(d, config.ffn),
        }
        if config.owner_of(layer) != layer:   # a KV-sharing layer projects q only
            del entry["k"], entry["v"]
        w.layers.append(entry)
    w.final_norm = np.ones(d, dtype=np.float32)
    w.lm_head = lin(config.vocab, d)
    w.rope_cos, w.rope_sin = rope_tables(config)
    for depth in config.head_dims:
        if depth != config.head_dim:
            w.rope_by_depth[depth] = rope_tables(config, depth)
    return w


class _DeviceLinear:
    def __init__(self, gpu: GpuContext, lin: Int4Linear):
        self.n, self.k = lin.n, lin.k
        self.w = gpu.upload(lin.packed)
        # fp16 scales (the benchmark configs) or f32 scales (the IR's companion tensors)
        self.scale_dtype = F16 if lin.scales.dtype == np.float16 else F32
        self.s = gpu.upload(np.ascontiguousarray(
            lin.scales, dtype=np.float16 if self.scale_dtype == F16 else np.float32))


def _stack_rows(*lins: Int4Linear) -> Int4Linear:
    """[a; b; ...] along the output rows (one launch for q, k and v)."""
    return Int4Linear(sum(l.n for l in lins), lins[0].k,
                      np.concatenate([l.packed for l in lins], axis=0),
                      np.concatenate([l.scales for l in lins], axis=0))


def _interleave_rows(a: Int4Linear, b: Int4Linear) -> Int4Linear:
    """Rows (2i, 2i+1) = (a_i, b_i): the layout of the fused gate/up epilogue."""
    packed = np.empty((a.n * 2, a.packed.shape[1]), dtype=np.uint8)
    packed[0::2], packed[1::2] = a.packed, b.packed
    scales = np.empty((a.n * 2, a.scales.shape[1]), dtype=a.scales.dtype)
    scales[0::2], scales[1::2] = a.scales, b.scales
    return Int4Linear(a.n * 2, a.k, packed, scales)


def _rope_pair_rows(lin: Int4Linear, head_dim: int) -> Int4Linear:
    """Rows of every head reordered to (0, D/2, 1, D/2 + 1, ...): the two halves of a rotation
    pair become neighbours, which is what the fused qkv launch expects for q and k."""
    half = head_dim // 2
    heads = lin.n // head_dim
    order = (np.arange(heads)[:, None, None] * head_dim
             + np.arange(half)[None, :, None] + np.array([0, half])[None, None, :]).reshape(-1)
    return Int4Linear(lin.n, lin.k, np.ascontiguousarray(lin.packed[order]),
                      np.ascontiguousarray(lin.scales[order]))


class LlamaDecoderSession:
    """Weights resident on the device + scratch activations for chunks of up to chunk_length
    rows.  io dtype selects f32 (the reference's semantic dtype) or fp16 activations; kv dtype
    the state-slot storage."""

    def __init__(self, gpu: GpuContext, weights: DecoderWeights, *, io_dtype: int = F32,
                 kv_dtype: int = F32, chunk_length: int = 128,
                 prefill_compute: int = COMPUTE_F32, fuse_decode: bool = True):
        self.gpu = gpu
        self.config = c = weights.config
        self.io_dtype, self.kv_dtype = io_dtype, kv_dtype
        self.io_np = np.float16 if io_dtype == F16 else np.float32
        self.eb = 2 if io_dtype == F16 else 4
        self.kv_eb = 2 if kv_dtype == F16 else 4
        self.chunk_length = chunk_length
        self.prefill_compute = prefill_compute
        self.half_activations = True  # fp16 copies of product-only activations (COMPUTE_F16)
        # One-row steps use the fused launches: rms_norm + [q;k;v], o + residual,
        # rms_norm + interleaved gate/up + silu*mul, down + residual.
        self.fuse_decode = fuse_decode
        self.embedding = gpu.upload(weights.embedding)
        self.layers = []
        # per-layer attention structure: head dim, owner of the K / V, readers of an owner
        self.spec = []
        for li in range(c.layers):
            depth, owner = c.depth_of(li), c.owner_of(li)
            readers = c.readers_of(li) if owner == li else []
            self.spec.append({"depth": depth, "hd": c.heads * depth, "kvd": c.kv_heads * depth,
                              "owner": owner, "last_reader": readers[-1] if readers else li,
                              "shared": len(readers) > 1, "half_scale": c.half_scale_of(li)})
        for li, lw in enumerate(weights.layers):
            owns = c.owner_of(li) == li
            names = ("q", "k", "v", "o", "gate", "up", "down") if owns else \
                ("q", "o", "gate", "up", "down")
            entry = {
                "attn_norm": gpu.upload(lw["attn_norm"]), "ffn_norm": gpu.upload(lw["ffn_norm"]),
                **{name: _DeviceLinear(gpu, lw[name]) for name in names},
            }
            if fuse_decode:
                depth = c.depth_of(li)
                if owns:
                    entry["qkv"] = _DeviceLinear(gpu, _stack_rows(
                        _rope_pair_rows(lw["q"], depth), _rope_pair_rows(lw["k"], depth), lw["v"]))
                else:   # a KV-sharing layer: the fused launch carries the q rows only
                    entry["qkv"] = _DeviceLinear(gpu, _rope_pair_rows(lw["q"], depth))
                entry["gate_up"] = _DeviceLinear(gpu, _interleave_rows(lw["gate"], lw["up"]))
            self.layers.append(entry)
        self.final_norm = gpu.upload(weights.final_norm)
        self.lm_head = _DeviceLinear(gpu, weights.lm_head)
        # RoPE tables, one pair per head dim
        self.rope = {depth: tuple(gpu.upload(t) for t in weights.rope_of(depth))
                     for depth in c.head_dims}
        m, d = chunk_length, c.d_model
        hd = max(sp["hd"] for sp in self.spec)
        kvd = max(sp["kvd"] for sp in self.spec)
        eb = self.eb
        a = gpu.alloc
        self.buf = {
            "ids": a(m * 4), "pos": a(m * 4), "h": a(m * d * eb), "xn": a(m * d * eb),
            "q": a(m * hd * eb), "k": a(m * kvd * eb), "v": a(m * kvd * eb),
            "qr": a(m * hd * eb), "kr": a(m * kvd * eb), "vt": a(m * kvd * eb),
            "att": a(m * hd * eb), "att2": a(m * hd * eb), "o": a(m * d * eb),
            "g": a(m * c.ffn * eb), "u": a(m * c.ffn * eb), "act": a(m * c.ffn * eb),
            "dn": a(m * d * eb), "logits": a(c.vocab * eb), "token": a(16),
            "qkv": a((hd + 2 * kvd) * eb), "qkr": a((hd + kvd) * eb),
            # per-workgroup argmax pairs of the head projection (8 bytes per 4 rows at most)
            "argmax_part": a((c.vocab + 3) // 4 * 8),
        }
        # An owner whose K / V other layers read keeps this step's rows in buffers of its own
        # until its last reader has run (the shared scratch above is reused by every layer).
        for li, sp in enumerate(self.spec):
            if sp["shared"]:
                self.buf[f"kr{li}"] = a(m * sp["kvd"] * eb)
                self.buf[f"vt{li}"] = a(m * sp["kvd"] * eb)
                self.buf[f"qkv{li}"] = a((sp["hd"] + 2 * sp["kvd"]) * eb)
        self.workspace: Optional[DeviceBuffer] = None
        self.logits_shape = (1, c.vocab)

    def close(self) -> None:
        """Free every device buffer of the session (weights, tables, scratch activations)."""
        for entry in self.layers:
            for value in entry.values():
                if isinstance(value, _DeviceLinear):
                    value.w.free()
                    value.s.free()
                else:
                    value.free()
        tables = [t for pair in self.rope.values() for t in pair]
        for buf in list(self.buf.values()) + [self.embedding, self.final_norm, self.lm_head.w,
                                              self.lm_head.s] + tables:
            buf.free()
        if self.workspace is not None:
            self.workspace.free()
            self.workspace = None
        self.layers, self.buf = [], {}

    # -- GreedySession surface ---------------------------------------------------------------
    def create_generation_context(self, *, capacity: int, chunk_length: int) -> GenerationContext:
        if chunk_length != self.chunk_length:
            raise ExecutionError(f"chunkLength {chunk_length} differs from the session's "
                                 f"{self.chunk_length}")
        c = self.config
        layers = range(c.layers)
        for li in layers:
            if c.window_of(li) > capacity:
                raise ExecutionError(f"layer {li}: window {c.window_of(li)} exceeds capacity "
                                     f"{capacity}")
        ctx = GenerationContext(self.gpu, layers=c.layers, kv_planes=c.kv_heads,
                                depth=c.head_dim, capacity=capacity, chunk_length=chunk_length,
                                kv_itemsize=self.kv_eb,
                                layer_depths=[c.depth_of(li) for li in layers],
                                layer_windows=[c.window_of(li) for li in layers],
                                layer_owners=[c.owner_of(li) for li in layers])
        need = max(self.gpu.attention_state_workspace(1, c.heads, c.kv_heads, 1, c.depth_of(li),
                                                      c.window_of(li), capacity)
                   for li in layers)
        if self.workspace is None or self.workspace.nbytes < need:
            if self.workspace is not None:
                self.workspace.free()
            self.workspace = self.gpu.alloc(need)
        return ctx

    def run(self, input_ids: np.ndarray, position_ids: np.ndarray, last_row: Optional[int], *,
            context: GenerationContext, query_length: int, want_logits: bool = False):
        """One run of the decode graph over a chunk of M rows, of which the first
        `query_length` are valid.  With `last_row` (the token-only exit of the reference's
        default asset) the head runs on that row alone: token [1, 1, 1] (and logits [1, V]).
        With `last_row=None` the session returns what the reference graph itself returns
        (tools/export-recipes/minicpm5/export_decode.py:14-22): the argmax of every row,
        [1, M, 1] (and logits [1, M, V]); rows past `query_length` are unspecified."""
        ids = np.ascontiguousarray(input_ids, dtype=np.int32)
        pos = np.ascontiguousarray(position_ids, dtype=np.int32)
        if ids.ndim != 2 or ids.shape[0] != 1 or pos.shape != ids.shape:
            raise ExecutionError(f"ids {list(ids.shape)} / positions {list(pos.shape)} are not "
                                 "[1, M]")
        m = ids.shape[1]
        past = context.begin_run(m, query_length)
        all_rows = last_row is None
        if not all_rows and not 0 <= last_row < query_length:
            raise ExecutionError(f"last_row {last_row} is outside the {query_length} valid rows")
        try:
            self.buf["ids"].upload(ids)
            self.buf["pos"].upload(pos)
            if all_rows and m > 1:
                self._forward(context, m, past, query_length, None, lengths=None)
                token = self.buf["tokens_all"].download(np.int32, (1, m, 1))
                logits = (self.buf["logits_all"].download(self.io_np, (1, m, self.config.vocab))
                          if want_logits else None)
            else:
                self._forward(context, m, past, query_length, 0 if all_rows else last_row,
                              lengths=None)
                token = self.buf["token"].download(np.int32, (1, 1, 1))
                shape = (1, 1, self.config.vocab) if all_rows else self.logits_shape
                logits = (self.buf["logits"].download(self.io_np, shape)
                          if want_logits else None)
        except KarumeError:
            context.poison()  # a state write may already have happened: no rollback
            raise
        context.advance(past, query_length)
        return (token, logits) if want_logits else token

    # -- one chunk ---------------------------------------------------------------------------
    def _linear(self, x, lin: _DeviceLinear, out, m: int) -> None:
        compute = self.prefill_compute if m > 16 else COMPUTE_F32
        self.gpu.linear_i4(x, lin.w, lin.s, None, out, m, lin.n, lin.k, self.config.group_size,
                           self.io_dtype, lin.scale_dtype, compute)

    def _forward(self, context: GenerationContext, m: int, past: int, query: int,
                 last_row: Optional[int], lengths: Optional[DeviceBuffer], ids: Optional[DeviceBuffer] = None,
                 step_end: Optional[tuple] = None) -> None:
        """`step_end` = (history, history_len): a replayed one-row step whose input row is
        already in the activation buffer (the previous step's exit wrote it) and whose exit
        also does the step's bookkeeping and the next step's embedding."""
        g, c, b, io = self.gpu, self.config, self.buf, self.io_dtype
        d = c.d_model
        if step_end is None:
            g.embedding(self.embedding, ids if ids is not None else b["ids"], b["h"], m, c.vocab,
                        d, F16, io)
        if m == 1 and self.fuse_decode:
            self._forward_fused_row(context, past, lengths, step_end)
            return
        if step_end is not None:
            raise ExecutionError("the fused step exit needs the fused one-row launches")
        if m > 16 and self.fuse_decode and self._rows_form_covers(m):
            self._forward_rows(context, m, past, query, lengths)
            self._head(last_row, m)
            return
        pending = {}   # owner layer -> (k rows, v rows) whose appends wait for the last reader
        for li, lw in enumerate(self.layers):
            sp = self.spec[li]
            depth, owner = sp["depth"], sp["owner"]
            cos, sin = self.rope[depth]
            g.rms_norm(b["h"], lw["attn_norm"], b["xn"], m, d, c.rms_eps, io)
            self._linear(b["xn"], lw["q"], b["q"], m)
            g.rope_half(b["q"], b["pos"], cos, sin, b["qr"], m, c.heads, depth, c.max_position,
                        True, io)
            if owner == li:
                # this step's K / V rows: in buffers of the layer's own when later layers read them
                kr = b[f"kr{li}"] if sp["shared"] else b["kr"]
                vt = b[f"vt{li}"] if sp["shared"] else (b["vt"] if m > 1 else b["v"])
                self._linear(b["xn"], lw["k"], b["k"], m)
                self._linear(b["xn"], lw["v"], b["v"], m)
                g.rope_half(b["k"], b["pos"], cos, sin, kr, m, c.kv_heads, depth, c.max_position,
                            True, io)
                if m > 1:
                    g.transpose_01(b["v"], vt, m, c.kv_heads, depth, io)
                elif sp["shared"]:
                    g.copy(vt, b["v"], self._copy_bytes(sp["kvd"] * self.eb))
                pending[li] = (kr, vt)
            kr, vt = pending[owner]
            spec = dict(chunk_rows=m, depth=depth, capacity=context.layer_capacity[li],
                        window=context.layer_window[li])
            if lengths is None:
                g.attention_state(b["qr"], kr, vt, context.slots_k[li], context.slots_v[li],
                                  b["att"], batch=1, heads=c.heads, kv_heads=c.kv_heads,
                                  half_scale=sp["half_scale"], past=past, query=query,
                                  io_dtype=io, kv_dtype=self.kv_dtype, workspace=self.workspace,
                                  **spec)
            else:
                g.attention_state_lengths(b["qr"], kr, vt, context.slots_k[li],
                                          context.slots_v[li], b["att"], batch=1, heads=c.heads,
                                          kv_heads=c.kv_heads, half_scale=sp["half_scale"],
                                          lengths=lengths, max_past=context.capacity - 1,
                                          io_dtype=io, kv_dtype=self.kv_dtype,
                                          workspace=self.workspace, **spec)
            # readers first, then the appends (docs/ir-v1.md:345-348): the append of a slot
            # follows the last layer that reads it
            if self.spec[owner]["last_reader"] == li:
                self._append_pair(context, owner, pending.pop(owner), m, past, query, lengths)
            if m > 1:
                g.transpose_01(b["att"], b["att2"], c.heads, m, depth, io)
                att = b["att2"]
            else:
                att = b["att"]
            self._linear(att, lw["o"], b["o"], m)
            g.add(b["h"], b["o"], b["h"], m * d, io)
            g.rms_norm(b["h"], lw["ffn_norm"], b["xn"], m, d, c.rms_eps, io)
            self._linear(b["xn"], lw["gate"], b["g"], m)
            self._linear(b["xn"], lw["up"], b["u"], m)
            g.silu_mul(b["g"], b["u"], b["act"], m * c.ffn, io)
            self._linear(b["act"], lw["down"], b["dn"], m)
            g.add(b["h"], b["dn"], b["h"], m * d, io)
        self._head(last_row, m)

    @staticmethod
    def _copy_bytes(nbytes: int) -> int:
        """Device copies move whole 16-byte pieces (every buffer here is allocated in them)."""
        return (nbytes + 15) // 16 * 16

    def _append_pair(self, context: GenerationContext, li: int, rows: tuple, m: int, past: int,
                     query: int, lengths: Optional[DeviceBuffer]) -> None:
        """state_append of this step's K and V rows to the slots of layer `li`."""
        g, c, io = self.gpu, self.config, self.io_dtype
        spec = dict(chunk_rows=m, depth=self.spec[li]["depth"],
                    capacity=context.layer_capacity[li], window=context.layer_window[li])
        for src, slot in ((rows[0], context.slots_k[li]), (rows[1], context.slots_v[li])):
            if lengths is None:
                g.state_append(src, slot, kv_planes=c.kv_heads, past=past, query=query,
                               x_dtype=io, slot_dtype=self.kv_dtype, **spec)
            else:
                g.state_append_lengths(src, slot, kv_planes=c.kv_heads, lengths=lengths,
                                       x_dtype=io, slot_dtype=self.kv_dtype, **spec)

    def _head(self, last_row: Optional[int], m: int = 1) -> None:
        """Token-only exit: the head runs on the last valid row only.  `last_row=None`: the
        head runs on all m rows of the chunk (the graph's own outputs)."""
        g, c, b, io = self.gpu, self.config, self.buf, self.io_dtype
        if last_row is None:
            if "logits_all" not in b or b["logits_all"].nbytes < m * c.vocab * self.eb:
                for name in ("logits_all", "tokens_all"):
                    if name in b:
                        b.pop(name).free()
                b["logits_all"] = g.alloc(self.chunk_length * c.vocab * self.eb)
                b["tokens_all"] = g.alloc(self.chunk_length * 4)
            g.rms_norm(b["h"], self.final_norm, b["xn"], m, c.d_model, c.rms_eps, io)
            self._linear(b["xn"], self.lm_head, b["logits_all"], m)
            g.argmax(b["logits_all"], b["tokens_all"], m, c.vocab, io)
            return
        row = b["h"].offset(last_row * c.d_model * self.eb)
        g.rms_norm(row, self.final_norm, b["xn"], 1, c.d_model, c.rms_eps, io)
        self._linear(b["xn"], self.lm_head, b["logits"], 1)
        g.argmax(b["logits"], b["token"], 1, c.vocab, io)

    def _rows_form_covers(self, m: int) -> bool:
        """The chunk-of-rows launches need groups of 64 codes or more, K a multiple of 32 and
        (their limit for the f32 class and for 32-bit element offsets) no more than 65536 rows."""
        c = self.config
        return (c.group_size >= 64 and c.d_model % 32 == 0 and c.ffn % 32 == 0
                and all(sp["hd"] % 32 == 0 for sp in self.spec) and m <= 65536)

    def _forward_rows(self, context: GenerationContext, m: int, past: int, query: int,
                      lengths: Optional[DeviceBuffer]) -> None:
        """A chunk of m > 16 rows, 7 launches a layer: the [q; k; v] projection writes roped,
        head-major q / k / v, the attention writes row-major and appends the chunk's K / V rows,
        the o and down projections add the residual in place, the gate/up projection applies
        silu * up.  (A KV-sharing layer projects and rotates q alone, in two launches.)"""
        from .runtime import EPILOGUE_SILU_PAIRS
        g, c, b, io = self.gpu, self.config, self.buf, self.io_dtype
        d, group, compute = c.d_model, c.group_size, self.prefill_compute
        # COMPUTE_F16 rounds the f32 activations of every product to fp16: the three activations
        # only a product reads (both norms' outputs, the attention's, silu(gate) * up) are then
        # written as fp16 by their producers — the same values, half the bytes for the products
        half = self.half_activations and compute == COMPUTE_F16 and io == F32
        xd = F16 if half else io
        pending = {}   # owner layer -> (k rows, v rows) whose appends wait for the last reader
        for li, lw in enumerate(self.layers):
            sp = self.spec[li]
            depth, owner = sp["depth"], sp["owner"]
            window = context.layer_window[li]
            cos, sin = self.rope[depth]
            spec = dict(chunk_rows=m, depth=depth, capacity=context.layer_capacity[li],
                        window=window)
            g.rms_norm_cast(b["h"], lw["attn_norm"], b["xn"], m, d, c.rms_eps, io, xd)
            if owner == li:
                kr = b[f"kr{li}"] if sp["shared"] else b["kr"]
                vt = b[f"vt{li}"] if sp["shared"] else b["vt"]
                lin = lw["qkv"]
                g.prefill_qkv(b["xn"], lin.w, lin.s, b["pos"], cos, sin, b["qr"], kr, vt, m=m,
                              heads=c.heads, kv_heads=c.kv_heads, depth=depth, k=d, group=group,
                              table_rows=c.max_position, io_dtype=io, scale_dtype=lin.scale_dtype,
                              compute=compute, x_dtype=xd)
                pending[li] = (kr, vt)
            else:
                lin = lw["q"]
                g.linear_i4_rows(b["xn"], lin.w, lin.s, b["q"], m, lin.n, lin.k, group,
                                 io_dtype=io, scale_dtype=lin.scale_dtype, compute=compute,
                                 x_dtype=xd)
                g.rope_half(b["q"], b["pos"], cos, sin, b["qr"], m, c.heads, depth,
                            c.max_position, True, io)
            kr, vt = pending[owner]
            last_reader = self.spec[owner]["last_reader"] == li
            att_half = half and depth in (64, 128, 256)
            if depth in (64, 128, 256):
                # attention + output permute in one launch; it also appends the chunk's rows when
                # it is the slot's last reader and no window can wrap (slot rows past.. are read
                # by nobody in that launch)
                fold = last_reader and window == 0
                g.attention_chunk(b["qr"], kr, vt, context.slots_k[li], context.slots_v[li],
                                  b["att2"], batch=1, heads=c.heads, kv_heads=c.kv_heads,
                                  half_scale=sp["half_scale"], past=past, query=query,
                                  lengths=lengths, io_dtype=io, kv_dtype=self.kv_dtype,
                                  row_major=True, append=fold, out_f16=att_half, **spec)
                if last_reader:
                    rows = pending.pop(owner)
                    if not fold:
                        self._append_pair(context, owner, rows, m, past, query, lengths)
            else:
                if lengths is None:
                    g.attention_state(b["qr"], kr, vt, context.slots_k[li], context.slots_v[li],
                                      b["att"], batch=1, heads=c.heads, kv_heads=c.kv_heads,
                                      half_scale=sp["half_scale"], past=past, query=query,
                                      io_dtype=io, kv_dtype=self.kv_dtype,
                                      workspace=self.workspace, **spec)
                else:
                    g.attention_state_lengths(b["qr"], kr, vt, context.slots_k[li],
                                              context.slots_v[li], b["att"], batch=1,
                                              heads=c.heads, kv_heads=c.kv_heads,
                                              half_scale=sp["half_scale"], lengths=lengths,
                                              max_past=context.capacity - 1, io_dtype=io,
                                              kv_dtype=self.kv_dtype, workspace=self.workspace,
                                              **spec)
                # readers first, then the appends (docs/ir-v1.md:345-348)
                if last_reader:
                    self._append_pair(context, owner, pending.pop(owner), m, past, query, lengths)
                g.transpose_01(b["att"], b["att2"], c.heads, m, depth, io)
            lin = lw["o"]
            g.linear_i4_rows(b["att2"], lin.w, lin.s, b["h"], m, lin.n, lin.k, group,
                             residual=b["h"], io_dtype=io, scale_dtype=lin.scale_dtype,
                             compute=compute, x_dtype=F16 if att_half else io)
            g.rms_norm_cast(b["h"], lw["ffn_norm"], b["xn"], m, d, c.rms_eps, io, xd)
            lin = lw["gate_up"]
            # (fp16 in and out: silu(gate) * up is computed on the f32 sums and rounded once)
            g.linear_i4_rows(b["xn"], lin.w, lin.s, b["act"], m, lin.n, lin.k, group,
                             io_dtype=xd, scale_dtype=lin.scale_dtype, compute=compute,
                             epilogue=EPILOGUE_SILU_PAIRS)
            lin = lw["down"]
            g.linear_i4_rows(b["act"], lin.w, lin.s, b["h"], m, lin.n, lin.k, group,
                             residual=b["h"], io_dtype=io, scale_dtype=lin.scale_dtype,
                             compute=compute, x_dtype=xd)

    def _replay_max_past(self, context: GenerationContext) -> int:
        """Largest pastLength the recorded step will be replayed with: sizes the attention
        launch (a short replay needs one split and takes the prefetching form)."""
        hint = getattr(self, "_replay_last_past", None)
        return context.capacity - 1 if hint is None else min(context.capacity - 1, hint)

    def _fused(self, x, lin: _DeviceLinear, out, **kw) -> None:
        self.gpu.linear_i4_fused(x, lin.w, lin.s, out, 1, lin.n, lin.k, self.config.group_size,
                                 io_dtype=self.io_dtype, scale_dtype=lin.scale_dtype, **kw)

    def _forward_fused_row(self, context: GenerationContext, past: int,
                           lengths: Optional[DeviceBuffer],
                           step_end: Optional[tuple] = None) -> None:
        """One decode row (M = Q = 1), 5 launches per layer instead of 16."""
        from .runtime import EPILOGUE_SILU_PAIRS
        g, c, b, io, eb = self.gpu, self.config, self.buf, self.io_dtype, self.eb
        step_rows = {}   # owner layer -> its [q_rot; k_rot; v] buffer of this step
        for li, lw in enumerate(self.layers):
            sp = self.spec[li]
            depth, owner, hd, kvd = sp["depth"], sp["owner"], sp["hd"], sp["kvd"]
            cos, sin = self.rope[depth]
            spec = dict(chunk_rows=1, depth=depth, capacity=context.layer_capacity[li],
                        window=context.layer_window[li])
            # rms_norm + [q; k; v] + rope of q and k + both appends in one launch; a one-row
            # step's attention never reads the slot row this writes (the row holds a column
            # outside every window of this step), so it may go first — also for the later
            # layers that read the same slots
            lin = lw["qkv"]
            owns = owner == li
            out = b[f"qkv{li}"] if sp["shared"] else b["qkv"]
            g.decode_qkv(b["h"], lin.w, lin.s, b["pos"], cos, sin, out,
                         context.slots_k[li] if owns else None,
                         context.slots_v[li] if owns else None, heads=c.heads,
                         kv_heads=c.kv_heads if owns else 0, depth=depth, k=lin.k,
                         group=c.group_size, table_rows=c.max_position,
                         capacity=context.layer_capacity[li], window=context.layer_window[li],
                         past=past, lengths=lengths, norm_weight=lw["attn_norm"],
                         norm_eps=c.rms_eps, io_dtype=io, scale_dtype=lin.scale_dtype,
                         kv_dtype=self.kv_dtype)
            if owns:
                step_rows[li] = out
            # the launch leaves [q_rot; k_rot; v] in one buffer (a sharing layer: q_rot alone)
            q_r = out
            kv = step_rows[owner]
            k_r, v_row = kv.offset(hd * eb), kv.offset((hd + kvd) * eb)
            if lengths is None:
                g.attention_state(q_r, k_r, v_row, context.slots_k[li], context.slots_v[li],
                                  b["att"], batch=1, heads=c.heads, kv_heads=c.kv_heads,
                                  half_scale=sp["half_scale"], past=past, query=1, io_dtype=io,
                                  kv_dtype=self.kv_dtype, workspace=self.workspace, **spec)
            else:
                g.attention_state_lengths(q_r, k_r, v_row, context.slots_k[li],
                                          context.slots_v[li], b["att"], batch=1, heads=c.heads,
                                          kv_heads=c.kv_heads, half_scale=sp["half_scale"],
                                          lengths=lengths, max_past=self._replay_max_past(context),
                                          io_dtype=io, kv_dtype=self.kv_dtype,
                                          workspace=self.workspace, **spec)
            self._fused(b["att"], lw["o"], b["h"], residual=b["h"])
            self._fused(b["h"], lw["gate_up"], b["act"], norm_weight=lw["ffn_norm"],
                        norm_eps=c.rms_eps, epilogue=EPILOGUE_SILU_PAIRS)
            self._fused(b["act"], lw["down"], b["h"], residual=b["h"])
        if step_end is None:
            self._fused(b["h"], self.lm_head, b["logits"], norm_weight=self.final_norm,
                        norm_eps=c.rms_eps)
            g.argmax(b["logits"], b["token"], 1, c.vocab, io)
            return
        # the exit of a replayed step, two launches: head projection with argmax partials, then
        # argmax + bookkeeping + the next step's embedding row (into the activation buffer)
        history, history_len = step_end
        lm = self.lm_head
        count = g.decode_head(b["h"], lm.w, lm.s, b["logits"], b["argmax_part"], lm.n, lm.k,
                              c.group_size, norm_weight=self.final_norm, norm_eps=c.rms_eps,
                              io_dtype=io, scale_dtype=lm.scale_dtype)
        g.decode_tail(b["argmax_part"], count, b["token"], lengths, history, history_len,
                      b["pos"], self.embedding, c.vocab, c.d_model, b["h"], table_dtype=F16,
                      out_dtype=io)

    # -- replayed decode ---------------------------------------------------------------------
    def decode_tokens(self, context: GenerationContext, first_token: int, count: int
                      ) -> List[int]:
        """Feed `first_token` at position context.past and generate `count` more tokens, one
        recorded decode step replayed `count` times; lengths, positions and the fed-back token
        stay on the device and the tokens are read back once at the end."""
        if count < 1:
            return []
        if context.window == 0 and context.past + count > context.capacity:
            raise ExecutionError(f"pastLength {context.past} + {count} steps exceeds capacity "
                                 f"{context.capacity}")
        if context.past + count > self.config.max_position:
            raise ExecutionError("the decode would run past the RoPE table")
        g, b = self.gpu, self.buf
        context.begin_run(1, 1)
        history = g.zeros(count * 4)
        graph = None
        try:
            # the token buffer doubles as the id input: argmax writes it, the next replay's
            # embedding reads it
            b["token"].upload(np.array([first_token, 0, 0, 0], dtype=np.int32))
            g.lengths_set(context.lengths, context.past, 1)
            self._replay_last_past = context.past + count - 1
            g.lengths_positions(context.lengths, b["pos"], 1)
            if self.fuse_decode:
                # the first step's input row; every replay's exit leaves the next one's
                g.embedding(self.embedding, b["token"], b["h"], 1, self.config.vocab,
                            self.config.d_model, F16, self.io_dtype)
                with g.record() as rec:
                    self._forward(context, 1, 0, 1, 0, lengths=context.lengths,
                                  step_end=(history, count))
            else:
                with g.record() as rec:
                    self._forward(context, 1, 0, 1, 0, lengths=context.lengths, ids=b["token"])
                    # token logged, lengths advanced, the next replay's position written
                    g.lengths_step_end(context.lengths, b["token"], history, count, b["pos"])
            graph = rec.graph
            for _ in range(count):
                graph.launch()
            state = context.lengths.download(np.uint32, (4,))
            tokens = history.download(np.int32, (count,))
        except KarumeError:
            context.poison()
            raise
        finally:
            self._replay_last_past = None
            if graph is not None:
                graph.destroy()
            history.free()
        if state[2] != 0:
            context.poison()
            raise ExecutionError("a decode step violated the run contract on the device "
                                 "(pastLength + queryLength exceeded the capacity)")
        context.past = int(state[0])
        return [int(t) for t in tokens]
