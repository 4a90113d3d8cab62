"""GPU parity of the decoder-layer glue ops and of the whole decode graph (prefill chunks,
one-row decode steps, replayed decode) against the CPU oracle."""
import numpy as np
import pytest

import helpers
import karume_amd as ka
from helpers import oracle
from karume_amd.decoder import LlamaConfig, LlamaDecoderSession, random_weights
from karume_amd.generation import generate_greedy, plan_prefill_chunks

pytestmark = pytest.mark.gpu


def test_rms_norm_golden_and_random(gpu_ctx):
    """atol 1e-6 rtol 1e-5 (the reference's golden gate,
    packages/runtime/tests/e2e_golden_test.ts:43)."""
    rng = np.random.default_rng(0)
    x = rng.normal(size=(7, 2048)).astype(np.float32) * 3 + 0.5
    w = rng.normal(size=2048).astype(np.float32)
    dx, dw = gpu_ctx.upload(x), gpu_ctx.upload(w)
    out = gpu_ctx.alloc(x.nbytes)
    gpu_ctx.rms_norm(dx, dw, out, 7, 2048, 1e-5)
    got = out.download(np.float32, x.shape)
    ok, fails, max_abs, _ = oracle.allclose(got, oracle.rms_norm(x, w, 1e-5), atol=1e-6, rtol=1e-5)
    assert ok, (fails, max_abs)


def test_rope_silu_add_embedding_argmax(gpu_ctx):
    rng = np.random.default_rng(1)
    rows, heads, d, table = 5, 3, 8, 16
    x = rng.normal(size=(rows, heads, d)).astype(np.float32)
    pos = np.array([3, 0, 15, 7, 7], dtype=np.int32)
    ang = rng.normal(size=(table, d))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    dx, dp, dc, ds = map(gpu_ctx.upload, (x, pos, cos, sin))
    out = gpu_ctx.alloc(x.nbytes)
    gpu_ctx.rope_half(dx, dp, dc, ds, out, rows, heads, d, table, True)
    got = out.download(np.float32, (heads, rows, d))
    want = np.stack([oracle.rope_half(x[r][None, :, None, :], cos[pos[r]:pos[r] + 1],
                                      sin[pos[r]:pos[r] + 1])[0, :, 0] for r in range(rows)],
                    axis=1)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))  # same roundings: bit-exact
    gpu_ctx.rope_half(dx, dp, dc, ds, out, rows, heads, d, table, False)
    assert np.array_equal(out.download(np.float32, x.shape), want.transpose(1, 0, 2))
    # a position outside the table is NaN, never a wrapped row
    bad = gpu_ctx.upload(np.array([16, 0, 0, 0, -1], dtype=np.int32))
    gpu_ctx.rope_half(dx, bad, dc, ds, out, rows, heads, d, table, False)
    got = out.download(np.float32, x.shape)
    assert np.all(np.isnan(got[0])) and np.all(np.isnan(got[4])) and not np.any(np.isnan(got[1:4]))

    g = np.linspace(-30, 30, 4099).astype(np.float32)
    u = rng.normal(size=g.size).astype(np.float32)
    dg, du = gpu_ctx.upload(g), gpu_ctx.upload(u)
    o = gpu_ctx.alloc(g.nbytes)
    gpu_ctx.silu_mul(dg, du, o, g.size)
    ok, fails, max_abs, _ = oracle.allclose(o.download(np.float32, g.shape),
                                            oracle.silu_mul(g, u), atol=1e-6, rtol=1e-5)
    assert ok, (fails, max_abs)
    gpu_ctx.add(dg, du, o, g.size)
    assert np.array_equal(o.download(np.float32, g.shape), g + u)

    table_w = rng.normal(size=(11, 6)).astype(np.float16)
    idx = np.array([10, 0, 3, 11, -1], dtype=np.int32)
    dt, di = gpu_ctx.upload(table_w), gpu_ctx.upload(idx)
    eo = gpu_ctx.alloc(5 * 6 * 4)
    gpu_ctx.embedding(dt, di, eo, 5, 11, 6, ka.F16, ka.F32)
    got = eo.download(np.float32, (5, 6))
    assert np.array_equal(got[:3], table_w[[10, 0, 3]].astype(np.float32))
    assert np.all(np.isnan(got[3:]))

    # argmax: ties -> smallest index, NaN is the maximum, all -inf -> 0
    # (packages/runtime/src/reference/ops.ts:520-560) and the golden rows with ties
    rows_x = np.full((5, 1000), -1.0, dtype=np.float32)
    rows_x[0, [700, 300]] = 5.0
    rows_x[1, [999, 2]] = np.nan
    rows_x[2, :] = -np.inf
    rows_x[3, 999] = 0.0
    rows_x[4, :] = rng.normal(size=1000)
    dxr = gpu_ctx.upload(rows_x)
    ao = gpu_ctx.alloc(5 * 4)
    gpu_ctx.argmax(dxr, ao, 5, 1000)
    got = ao.download(np.int32, (5,))
    assert got.tolist() == [300, 2, 0, 999, int(oracle.argmax(rows_x[4:5])[0, 0])]


@pytest.mark.parametrize("io,kv", [(ka.F32, ka.F32), (ka.F32, ka.F16), (ka.F16, ka.F16)])
@pytest.mark.parametrize("window,past", [(0, 5), (4, 9), (0, 0)])
def test_decode_rope_append_equals_rope_then_appends(gpu_ctx, io, kv, window, past):
    """The one-launch decode row is bit-identical to krm_rope_half + two krm_state_append,
    with a host past and with device lengths; a violated contract appends nothing."""
    rng = np.random.default_rng(7 + past)
    heads, kv_heads, d, table, cap = 6, 2, 16, 32, 12
    io_np = np.float32 if io == ka.F32 else np.float16
    kv_np = np.float32 if kv == ka.F32 else np.float16
    qkv = rng.normal(size=(heads + 2 * kv_heads, d)).astype(io_np)
    ang = rng.normal(size=(table, d))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    pos = np.array([past], dtype=np.int32)
    slot0_k = rng.normal(size=(kv_heads, cap, d)).astype(kv_np)
    slot0_v = rng.normal(size=(kv_heads, cap, d)).astype(kv_np)
    dq, dp, dc, ds = map(gpu_ctx.upload, (qkv, pos, cos, sin))

    # separate launches
    ref_qk = gpu_ctx.alloc((heads + kv_heads) * d * qkv.itemsize)
    ref_k, ref_v = gpu_ctx.upload(slot0_k), gpu_ctx.upload(slot0_v)
    gpu_ctx.rope_half(dq, dp, dc, ds, ref_qk, 1, heads + kv_heads, d, table, True, io)
    spec = dict(kv_planes=kv_heads, chunk_rows=1, depth=d, capacity=cap, window=window,
                x_dtype=io, slot_dtype=kv)
    gpu_ctx.state_append(ref_qk.offset(heads * d * qkv.itemsize), ref_k, past=past, query=1, **spec)
    gpu_ctx.state_append(dq.offset((heads + kv_heads) * d * qkv.itemsize), ref_v, past=past,
                         query=1, **spec)
    want_qk = ref_qk.download(io_np, (heads + kv_heads, d))
    want_k, want_v = ref_k.download(kv_np, slot0_k.shape), ref_v.download(kv_np, slot0_v.shape)
    row = past % window if window else past
    assert not np.array_equal(want_k[:, row], slot0_k[:, row])

    lengths = gpu_ctx.zeros(16)
    for dyn in (False, True):
        got_qk = gpu_ctx.zeros((heads + kv_heads) * d * qkv.itemsize)
        got_k, got_v = gpu_ctx.upload(slot0_k), gpu_ctx.upload(slot0_v)
        if dyn:
            gpu_ctx.lengths_set(lengths, past, 1)
        gpu_ctx.decode_rope_append(dq, dp, dc, ds, got_qk, got_k, got_v, heads=heads,
                                   kv_heads=kv_heads, depth=d, table_rows=table, capacity=cap,
                                   window=window, past=0 if dyn else past,
                                   lengths=lengths if dyn else None, io_dtype=io, kv_dtype=kv)
        assert got_qk.download(io_np, want_qk.shape).tobytes() == want_qk.tobytes()
        assert got_k.download(kv_np, want_k.shape).tobytes() == want_k.tobytes()
        assert got_v.download(kv_np, want_v.shape).tobytes() == want_v.tobytes()
    assert lengths.download(np.uint32, (4,))[2] == 0

    if window == 0:
        # past = capacity: the host form refuses, the device form raises the fault word and
        # leaves both slots untouched
        with pytest.raises(ka.ExecutionError):
            gpu_ctx.decode_rope_append(dq, dp, dc, ds, got_qk, got_k, got_v, heads=heads,
                                       kv_heads=kv_heads, depth=d, table_rows=table,
                                       capacity=cap, past=cap, io_dtype=io, kv_dtype=kv)
        clean_k, clean_v = gpu_ctx.upload(slot0_k), gpu_ctx.upload(slot0_v)
        gpu_ctx.lengths_set(lengths, cap, 1)
        gpu_ctx.decode_rope_append(dq, dp, dc, ds, got_qk, clean_k, clean_v, heads=heads,
                                   kv_heads=kv_heads, depth=d, table_rows=table, capacity=cap,
                                   lengths=lengths, io_dtype=io, kv_dtype=kv)
        assert lengths.download(np.uint32, (4,))[2] == 1
        assert clean_k.download(kv_np, slot0_k.shape).tobytes() == slot0_k.tobytes()
        assert clean_v.download(kv_np, slot0_v.shape).tobytes() == slot0_v.tobytes()


@pytest.mark.parametrize("io,kv", [(ka.F32, ka.F32), (ka.F32, ka.F16), (ka.F16, ka.F16)])
@pytest.mark.parametrize("window,past,k", [(0, 5, 256), (4, 9, 2048), (0, 0, 4096)])
def test_decode_qkv_equals_linear_rope_appends(gpu_ctx, io, kv, window, past, k):
    """krm_decode_qkv (rms_norm + [q;k;v] + rope + appends, pair-interleaved q/k rows) writes
    the same bits as krm_linear_i4_fused + krm_rope_half + two krm_state_append."""
    from karume_amd.decoder import Int4Linear, _rope_pair_rows, _stack_rows
    rng = np.random.default_rng(11 + past)
    heads, kv_heads, d, table, cap, group = 4, 2, 32, 16, 12, 128
    io_np = np.float32 if io == ka.F32 else np.float16
    kv_np = np.float32 if kv == ka.F32 else np.float16
    n = (heads + 2 * kv_heads) * d
    packed, _codes, scales = helpers.synthetic_int4(rng, n, k, group)
    packed = packed.reshape(n, k // 2)
    x = rng.normal(size=(1, k)).astype(io_np)
    norm_w = rng.normal(1.0, 0.1, size=k).astype(np.float32)
    ang = rng.normal(size=(table, d))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    slot0_k = rng.normal(size=(kv_heads, cap, d)).astype(kv_np)
    slot0_v = rng.normal(size=(kv_heads, cap, d)).astype(kv_np)
    dx, dn, dc, ds = map(gpu_ctx.upload, (x, norm_w, cos, sin))
    dp = gpu_ctx.upload(np.array([past], dtype=np.int32))
    eb = x.itemsize
    hq, hk = heads * d, kv_heads * d

    # separate launches on the natural row order
    dw, dsc = gpu_ctx.upload(packed), gpu_ctx.upload(scales)
    qkv = gpu_ctx.alloc(n * eb)
    gpu_ctx.linear_i4_fused(dx, dw, dsc, qkv, 1, n, k, group, io_dtype=io, scale_dtype=ka.F16,
                            norm_weight=dn, norm_eps=1e-5)
    want = gpu_ctx.alloc(n * eb)
    gpu_ctx.rope_half(qkv, dp, dc, ds, want, 1, heads + kv_heads, d, table, True, io)
    gpu_ctx.copy(want.offset((hq + hk) * eb), qkv.offset((hq + hk) * eb), hk * eb)
    ref_k, ref_v = gpu_ctx.upload(slot0_k), gpu_ctx.upload(slot0_v)
    spec = dict(kv_planes=kv_heads, chunk_rows=1, depth=d, capacity=cap, window=window,
                x_dtype=io, slot_dtype=kv)
    gpu_ctx.state_append(want.offset(hq * eb), ref_k, past=past, query=1, **spec)
    gpu_ctx.state_append(want.offset((hq + hk) * eb), ref_v, past=past, query=1, **spec)
    want_row = want.download(io_np, (n,))
    want_k, want_v = ref_k.download(kv_np, slot0_k.shape), ref_v.download(kv_np, slot0_v.shape)

    # one launch on the pair-interleaved rows
    def part(lo, hi):
        return Int4Linear(hi - lo, k, packed[lo:hi], scales[lo:hi])
    fused = _stack_rows(_rope_pair_rows(part(0, hq), d), _rope_pair_rows(part(hq, hq + hk), d),
                        part(hq + hk, n))
    fw, fs = gpu_ctx.upload(fused.packed), gpu_ctx.upload(fused.scales)
    lengths = gpu_ctx.zeros(16)
    for dyn in (False, True):
        got = gpu_ctx.zeros(n * eb)
        got_k, got_v = gpu_ctx.upload(slot0_k), gpu_ctx.upload(slot0_v)
        if dyn:
            gpu_ctx.lengths_set(lengths, past, 1)
        gpu_ctx.decode_qkv(dx, fw, fs, dp, dc, ds, got, got_k, got_v, heads=heads,
                           kv_heads=kv_heads, depth=d, k=k, group=group, table_rows=table,
                           capacity=cap, window=window, past=0 if dyn else past,
                           lengths=lengths if dyn else None, norm_weight=dn, norm_eps=1e-5,
                           io_dtype=io, scale_dtype=ka.F16, kv_dtype=kv)
        assert got.download(io_np, (n,)).tobytes() == want_row.tobytes()
        assert got_k.download(kv_np, want_k.shape).tobytes() == want_k.tobytes()
        assert got_v.download(kv_np, want_v.shape).tobytes() == want_v.tobytes()
    assert lengths.download(np.uint32, (4,))[2] == 0
    if window == 0:
        with pytest.raises(ka.ExecutionError):
            gpu_ctx.decode_qkv(dx, fw, fs, dp, dc, ds, got, got_k, got_v, heads=heads,
                               kv_heads=kv_heads, depth=d, k=k, group=group, table_rows=table,
                               capacity=cap, past=cap, io_dtype=io, scale_dtype=ka.F16,
                               kv_dtype=kv)
        clean_k = gpu_ctx.upload(slot0_k)
        gpu_ctx.lengths_set(lengths, cap, 1)
        gpu_ctx.decode_qkv(dx, fw, fs, dp, dc, ds, got, clean_k, got_v, heads=heads,
                           kv_heads=kv_heads, depth=d, k=k, group=group, table_rows=table,
                           capacity=cap, lengths=lengths, io_dtype=io, scale_dtype=ka.F16,
                           kv_dtype=kv)
        assert lengths.download(np.uint32, (4,))[2] == 1
        assert clean_k.download(kv_np, slot0_k.shape).tobytes() == slot0_k.tobytes()


def test_transpose(gpu_ctx):
    x = np.arange(3 * 5 * 4, dtype=np.float32).reshape(3, 5, 4)
    dx = gpu_ctx.upload(x)
    out = gpu_ctx.alloc(x.nbytes)
    gpu_ctx.transpose_01(dx, out, 3, 5, 4)
    assert np.array_equal(out.download(np.float32, (5, 3, 4)), x.transpose(1, 0, 2))


SMALL = LlamaConfig(layers=2, d_model=256, ffn=384, heads=8, kv_heads=2, head_dim=32, vocab=512,
                    group_size=128, max_position=64)


@pytest.mark.parametrize("io,kv,atol", [(ka.F32, ka.F32, 2e-4), (ka.F16, ka.F16, 0.15)])
def test_decoder_chain_matches_full_reforward(gpu_ctx, io, kv, atol):
    """Prefill in chunks of 8 (last chunk padded), then one-row decode steps, teacher-forced
    with a fixed id sequence; the logits of every run's last valid row equal the oracle's full
    re-forward without a KV cache.  f32 activations: atol 2e-4 on logits of size ~10 (the
    reference gates real-model logits at atol 1e-3, packages/runtime/tests/
    e2e_minicpm5_test.ts:35-62).  fp16 activations and KV: atol 0.15 (fp16 residual stream)."""
    weights = random_weights(SMALL, seed=4)
    rng = np.random.default_rng(9)
    ids = rng.integers(0, SMALL.vocab, size=30).astype(np.int32)
    want = helpers.oracle_decoder_logits(weights, ids)
    session = LlamaDecoderSession(gpu_ctx, weights, io_dtype=io, kv_dtype=kv, chunk_length=8)
    ctx = session.create_generation_context(capacity=64, chunk_length=8)
    worst = 0.0
    prompt_len = 19
    for chunk in plan_prefill_chunks(prompt_len, 8):
        n = chunk.query_length
        cid = np.zeros((1, 8), dtype=np.int32)
        cpos = np.zeros((1, 8), dtype=np.int32)
        cid[0, :n] = ids[chunk.position:chunk.position + n]
        cpos[0, :n] = np.arange(chunk.position, chunk.position + n)
        token, logits = session.run(cid, cpos, n - 1, context=ctx, query_length=n,
                                    want_logits=True)
        row = chunk.position + n - 1
        worst = max(worst, float(np.max(np.abs(logits.astype(np.float32)[0] - want[row]))))
    for pos in range(prompt_len, 30):
        token, logits = session.run(ids[pos:pos + 1][None], np.array([[pos]], dtype=np.int32), 0,
                                    context=ctx, query_length=1, want_logits=True)
        err = float(np.max(np.abs(logits.astype(np.float32)[0] - want[pos])))
        worst = max(worst, err)
        if io == ka.F32:
            margin = np.sort(want[pos])[-1] - np.sort(want[pos])[-2]
            if margin > 2 * atol:
                assert int(token[0, 0, 0]) == int(np.argmax(want[pos]))
    assert ctx.past == 30
    assert worst <= atol, worst
    ctx.dispose()


def test_greedy_loop_and_replayed_decode_agree(gpu_ctx):
    """generate_greedy (a read-back per step) and decode_tokens (one recorded step replayed,
    lengths and token feedback on the device) produce the same token sequence, and it equals
    the oracle's greedy continuation wherever the oracle's top-1/top-2 margin exceeds twice the
    logits tolerance."""
    weights = random_weights(SMALL, seed=5)
    prompt = [int(t) for t in np.random.default_rng(3).integers(0, SMALL.vocab, size=11)]
    session = LlamaDecoderSession(gpu_ctx, weights, io_dtype=ka.F32, kv_dtype=ka.F32,
                                  chunk_length=8)
    new = 12
    stepwise = generate_greedy(session, prompt=prompt, max_new_tokens=new, chunk_length=8,
                               max_position=SMALL.max_position)
    # replayed: prefill through run(), then the rest on the device
    ctx = session.create_generation_context(capacity=SMALL.max_position, chunk_length=8)
    token = None
    for chunk in plan_prefill_chunks(len(prompt), 8):
        n = chunk.query_length
        cid = np.zeros((1, 8), dtype=np.int32)
        cpos = np.zeros((1, 8), dtype=np.int32)
        cid[0, :n] = prompt[chunk.position:chunk.position + n]
        cpos[0, :n] = np.arange(chunk.position, chunk.position + n)
        token = session.run(cid, cpos, n - 1, context=ctx, query_length=n)
    first = int(token[0, 0, 0])
    replayed = [first] + session.decode_tokens(ctx, first, new - 1)
    assert replayed == stepwise
    assert ctx.past == len(prompt) + new - 1
    ctx.dispose()
    # oracle greedy with margins
    seq = list(prompt)
    for step in range(new):
        logits = helpers.oracle_decoder_logits(weights, np.array(seq, dtype=np.int32))[-1]
        top = np.sort(logits)
        if top[-1] - top[-2] <= 4e-4:
            break  # the continuation is not strongly determined from here on
        assert stepwise[step] == int(np.argmax(logits)), step
        seq.append(stepwise[step])


def test_all_rows_exit_returns_what_the_graph_returns(gpu_ctx):
    """`last_row=None`: the session returns the decode graph's own outputs, logits [1, M, V] and
    token [1, M, 1] (tools/export-recipes/minicpm5/export_decode.py:14-22).  A padded chunk (5 of
    8 rows valid) then a padded second chunk and a one-row step: every valid row's logits equal
    the oracle's full re-forward (atol 2e-4, the gate of the last-row form) and its token the
    oracle's argmax wherever the margin exceeds twice that; pad rows are unspecified.  The
    greedy loop gives the same tokens through either exit."""
    weights = random_weights(SMALL, seed=8)
    ids = np.random.default_rng(12).integers(0, SMALL.vocab, size=12).astype(np.int32)
    want = helpers.oracle_decoder_logits(weights, ids)
    session = LlamaDecoderSession(gpu_ctx, weights, chunk_length=8)
    ctx = session.create_generation_context(capacity=32, chunk_length=8)
    position = 0
    for n, m in ((5, 8), (6, 8), (1, 1)):
        cid = np.zeros((1, m), dtype=np.int32)
        cpos = np.zeros((1, m), dtype=np.int32)
        cid[0, :n] = ids[position:position + n]
        cpos[0, :n] = np.arange(position, position + n)
        token, logits = session.run(cid, cpos, None, context=ctx, query_length=n,
                                    want_logits=True)
        assert token.shape == (1, m, 1) and token.dtype == np.int32
        assert logits.shape == (1, m, SMALL.vocab)
        for row in range(n):
            ref = want[position + row]
            assert float(np.max(np.abs(logits[0, row] - ref))) <= 2e-4, (position, row)
            top = np.sort(ref)
            if top[-1] - top[-2] > 4e-4:
                assert int(token[0, row, 0]) == int(np.argmax(ref)), (position, row)
        position += n
    assert ctx.past == 12
    ctx.dispose()
    prompt = [int(t) for t in ids[:11]]
    by_last_row = generate_greedy(session, prompt=prompt, max_new_tokens=6, chunk_length=8,
                                  max_position=SMALL.max_position)
    by_all_rows = generate_greedy(session, prompt=prompt, max_new_tokens=6, chunk_length=8,
                                  max_position=SMALL.max_position, last_row=False)
    assert by_all_rows == by_last_row
    session.close()


@pytest.mark.parametrize("io,n,k", [(np.float32, 32000, 2048), (np.float32, 1003, 512),
                                    (np.float16, 4096, 4096), (np.float32, 70000, 256)])
def test_decode_head_and_tail_equal_the_separate_ops(gpu_ctx, io, n, k):
    """krm_decode_head + krm_decode_tail against the four launches they stand for: the logits
    are those of krm_linear_i4_fused bit for bit, the token is krm_argmax of them, the
    bookkeeping is krm_lengths_step_end's and the next row is krm_embedding's."""
    ctx = gpu_ctx
    rng = np.random.default_rng(n + k)
    g, hidden = 128, 96
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, g)
    x = rng.normal(size=(1, k)).astype(io)
    norm = rng.normal(size=k).astype(np.float32)
    table = rng.normal(size=(n, hidden)).astype(np.float16)
    dx, dw, ds, dn, dt = (ctx.upload(a) for a in (x, packed, scale, norm, table))
    code = ka.dtype_code(io)
    eb = np.dtype(io).itemsize
    logits_a, logits_b = ctx.alloc(n * eb), ctx.alloc(n * eb)
    ctx.linear_i4_fused(dx, dw, ds, logits_a, 1, n, k, g, norm_weight=dn, norm_eps=1e-5,
                        io_dtype=code, scale_dtype=ka.F16)
    token_a = ctx.alloc(16)
    ctx.argmax(logits_a, token_a, 1, n, code)
    partials = ctx.alloc((n + 3) // 4 * 8)
    count = ctx.decode_head(dx, dw, ds, logits_b, partials, n, k, g, norm_weight=dn,
                            norm_eps=1e-5, io_dtype=code, scale_dtype=ka.F16)
    assert 1 <= count <= (n + 3) // 4
    assert logits_b.download(io, (n,)).tobytes() == logits_a.download(io, (n,)).tobytes()
    lengths = ctx.alloc(16)
    ctx.lengths_set(lengths, 41, 1)
    history = ctx.zeros(8 * 4)
    token_b, pos, row = ctx.alloc(16), ctx.alloc(16), ctx.alloc(hidden * 4)
    for step in range(2):  # two steps in a row: the log slot and the position advance
        ctx.decode_tail(partials, count, token_b, lengths, history, 8, pos, dt, n, hidden, row,
                        table_dtype=ka.F16, out_dtype=ka.F32)
    want = int(token_a.download(np.int32, (1,))[0])
    assert int(token_b.download(np.int32, (1,))[0]) == want
    assert list(history.download(np.int32, (8,))[:3]) == [want, want, 0]
    assert list(lengths.download(np.uint32, (4,))) == [43, 1, 0, 2]
    assert int(pos.download(np.int32, (1,))[0]) == 43
    assert np.array_equal(row.download(np.float32, (hidden,)), table[want].astype(np.float32))
    for b in (dx, dw, ds, dn, dt, logits_a, logits_b, token_a, token_b, partials, lengths,
              history, pos, row):
        b.free()


def test_decode_tail_orders_pairs_like_argmax(gpu_ctx):
    """The tail's merge on hand-made pairs: ties go to the smallest row, NaN is the maximum
    (the smallest row among NaNs), a row of -inf gives row 0; a faulted step keeps pastLength
    (packages/runtime/src/kernels/argmax.ts:16-34, generation-context.ts:576-591)."""
    ctx = gpu_ctx
    hidden = 8
    table = np.arange(6000 * hidden, dtype=np.float32).reshape(6000, hidden)
    dt = ctx.upload(table)

    def run(values, rows, fault=0):
        pairs = np.empty((len(values), 2), dtype=np.uint32)
        pairs[:, 0] = np.asarray(values, dtype=np.float32).view(np.uint32)
        pairs[:, 1] = rows
        dp = ctx.upload(pairs)
        lengths = ctx.upload(np.array([10, 1, fault, 0], dtype=np.uint32))
        history, token, pos, row = ctx.zeros(16), ctx.alloc(16), ctx.alloc(16), ctx.alloc(hidden * 4)
        ctx.decode_tail(dp, len(values), token, lengths, history, 4, pos, dt, 6000, hidden, row,
                        table_dtype=ka.F32, out_dtype=ka.F32)
        out = (int(token.download(np.int32, (1,))[0]), list(lengths.download(np.uint32, (4,))),
               int(pos.download(np.int32, (1,))[0]), row.download(np.float32, (hidden,)))
        for b in (dp, lengths, history, token, pos, row):
            b.free()
        return out

    many = 5000  # more pairs than threads: the strided walk and the tree both take part
    rows = np.arange(many, dtype=np.uint32)[::-1].copy()   # descending rows: order must not matter
    values = np.full(many, -1.0, dtype=np.float32)
    values[[100, 4000]] = 7.0                               # rows 4899 and 999 tie
    token, lengths, pos, row = run(values, rows)
    assert token == 999 and lengths == [11, 1, 0, 1] and pos == 11
    assert np.array_equal(row, table[999])
    values[[7, 4500]] = np.nan                              # rows 4992 and 499
    assert run(values, rows)[0] == 499
    assert run(np.full(many, -np.inf, dtype=np.float32), rows)[0] == 0
    # workgroups without a row leave {-inf, 0xffffffff}: they never win
    assert run([-np.inf, -np.inf, -np.inf], [0xFFFFFFFF, 5, 0xFFFFFFFF])[0] == 5
    token, lengths, pos, _ = run(values, rows, fault=1)
    assert lengths == [10, 1, 1, 1] and pos == 10          # the fault keeps pastLength


def test_fused_and_separate_decode_launches_agree(gpu_ctx):
    """The fused one-row step (5 launches per layer) and the op-by-op step (16 launches) give
    logits within 1e-4 of each other and the same tokens on a teacher-forced sequence."""
    weights = random_weights(SMALL, seed=7)
    ids = np.random.default_rng(2).integers(0, SMALL.vocab, size=14).astype(np.int32)
    outs = []
    for fuse in (True, False):
        session = LlamaDecoderSession(gpu_ctx, weights, chunk_length=8, fuse_decode=fuse)
        ctx = session.create_generation_context(capacity=32, chunk_length=8)
        rows = []
        for pos in range(14):
            _tok, logits = session.run(ids[pos:pos + 1][None], np.array([[pos]], dtype=np.int32),
                                       0, context=ctx, query_length=1, want_logits=True)
            rows.append(logits[0].copy())
        outs.append(np.stack(rows))
        ctx.dispose()
    assert np.max(np.abs(outs[0] - outs[1])) <= 1e-4
    want = helpers.oracle_decoder_logits(weights, ids)
    assert np.max(np.abs(outs[0] - want)) <= 2e-4


def test_context_capacity_and_poison(gpu_ctx):
    """Capacity overflow is rejected before launch and leaves the context usable; a context is
    unusable after dispose (packages/runtime/tests/gpu_state_execution_test.ts:670-712)."""
    weights = random_weights(SMALL, seed=6)
    session = LlamaDecoderSession(gpu_ctx, weights, chunk_length=8)
    ctx = session.create_generation_context(capacity=8, chunk_length=8)
    ids = np.arange(8, dtype=np.int32)[None]
    session.run(ids, ids, 7, context=ctx, query_length=8)
    with pytest.raises(ka.ExecutionError):
        session.run(ids[:, :1], np.array([[8]], dtype=np.int32), 0, context=ctx, query_length=1)
    assert ctx.past == 8 and not ctx.poisoned
    ctx.rewind(4)
    session.run(ids[:, :1], np.array([[4]], dtype=np.int32), 0, context=ctx, query_length=1)
    assert ctx.past == 5
    with pytest.raises(ka.ExecutionError):
        session.decode_tokens(ctx, 1, 10)
    ctx.dispose()
    with pytest.raises(ka.KarumeError):
        session.run(ids[:, :1], ids[:, :1], 0, context=ctx, query_length=1)


def test_lengths_step_end_equals_the_three_launches(gpu_ctx):
    """krm_lengths_step_end = log_token + advance + positions (one row), clean and faulted."""
    for fault in (0, 1):
        state = np.array([41, 1, fault, 2], dtype=np.uint32)
        token = gpu_ctx.upload(np.array([777, 0, 0, 0], dtype=np.int32))
        outs = []
        for fused in (False, True):
            lengths = gpu_ctx.upload(state.copy())
            history = gpu_ctx.upload(np.full(4, -1, dtype=np.int32))
            pos = gpu_ctx.upload(np.full(4, -5, dtype=np.int32))
            if fused:
                gpu_ctx.lengths_step_end(lengths, token, history, 4, pos)
            else:
                gpu_ctx.lengths_log_token(lengths, token, history, 4)
                gpu_ctx.lengths_advance(lengths)
                gpu_ctx.lengths_positions(lengths, pos, 1)
            outs.append((lengths.download(np.uint32, (4,)).tolist(),
                         history.download(np.int32, (4,)).tolist(),
                         pos.download(np.int32, (4,)).tolist()))
        assert outs[0] == outs[1]
        assert outs[1][0][0] == (41 if fault else 42) and outs[1][1][2] == 777


def test_session_from_a_model_file_equals_session_from_arrays(gpu_ctx):
    """A decoder written out as a Karume model file (safetensors + karume_ir graph in the decode
    recipe's node order), read back with open_model / DecoderWeights.from_model, prefills and
    decodes to the same logits bits and tokens as the session built from the arrays (the file
    carries f32 scale companions, the arrays fp16 ones: the same numbers)."""
    from karume_amd.decoder import DecoderWeights
    from model_file import decoder_model_file

    weights = random_weights(SMALL, seed=21)
    loaded = DecoderWeights.from_model(ka.open_model(decoder_model_file(weights)))
    assert loaded.config == SMALL
    ids = np.random.default_rng(8).integers(0, SMALL.vocab, size=13).astype(np.int32)
    results = []
    for w in (weights, loaded):
        session = LlamaDecoderSession(gpu_ctx, w, io_dtype=ka.F32, kv_dtype=ka.F32, chunk_length=8)
        ctx = session.create_generation_context(capacity=SMALL.max_position, chunk_length=8)
        rows = []
        for chunk in plan_prefill_chunks(11, 8):
            n = chunk.query_length
            cid, cpos = np.zeros((1, 8), dtype=np.int32), np.zeros((1, 8), dtype=np.int32)
            cid[0, :n] = ids[chunk.position:chunk.position + n]
            cpos[0, :n] = np.arange(chunk.position, chunk.position + n)
            rows.append(session.run(cid, cpos, n - 1, context=ctx, query_length=n,
                                    want_logits=True))
        for pos in (11, 12):
            rows.append(session.run(ids[pos:pos + 1][None], np.array([[pos]], dtype=np.int32), 0,
                                    context=ctx, query_length=1, want_logits=True))
        tokens = session.decode_tokens(ctx, int(rows[-1][0][0, 0, 0]), 5)
        results.append((rows, tokens))
        ctx.dispose()
        session.close()
    (rows_a, tokens_a), (rows_b, tokens_b) = results
    assert tokens_a == tokens_b
    for (tok_a, log_a), (tok_b, log_b) in zip(rows_a, rows_b):
        assert np.array_equal(tok_a, tok_b)
        assert log_a.tobytes() == log_b.tobytes()


@pytest.mark.parametrize("io,compute,m", [(ka.F32, ka.COMPUTE_F32, 40), (ka.F32, ka.COMPUTE_F16, 128),
                                          (ka.F16, ka.COMPUTE_F16, 33), (ka.F32, ka.COMPUTE_F32, 5)])
def test_prefill_qkv_equals_linear_rope_transpose(gpu_ctx, io, compute, m):
    """krm_prefill_qkv (fused [q;k;v] projection of a chunk on pair-interleaved rows + RoPE,
    head-major) writes the same bits as krm_linear_i4_rows on the natural rows followed by
    krm_rope_half (to head-major) for q and k and krm_transpose_01 for v; a position outside
    the table gives NaN in that row of q and k only."""
    from karume_amd.decoder import Int4Linear, _rope_pair_rows, _stack_rows
    rng = np.random.default_rng(100 + m)
    heads, kv_heads, d, table, k, group = 8, 2, 64, 200, 512, 128
    io_np = np.float32 if io == ka.F32 else np.float16
    eb = np.dtype(io_np).itemsize
    hq, hk = heads * d, kv_heads * d
    n = hq + 2 * hk
    packed, _codes, scales = helpers.synthetic_int4(rng, n, k, group)
    packed = packed.reshape(n, k // 2)
    x = rng.normal(size=(m, k)).astype(io_np)
    ang = rng.normal(size=(table, d))
    cos, sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
    pos = rng.integers(0, table, size=m).astype(np.int32)
    pos[m // 2] = table + 3                       # outside the table
    dx, dc, ds, dp = map(gpu_ctx.upload, (x, cos, sin, pos))

    def linear(lo, hi):
        out = gpu_ctx.alloc(m * (hi - lo) * eb)
        gpu_ctx.linear_i4_rows(dx, gpu_ctx.upload(packed[lo:hi]), gpu_ctx.upload(scales[lo:hi]), out,
                               m, hi - lo, k, group, io_dtype=io, scale_dtype=ka.F16,
                               compute=compute)
        return out
    q, kk, v = linear(0, hq), linear(hq, hq + hk), linear(hq + hk, n)
    want_q, want_k, want_v = (gpu_ctx.alloc(m * hq * eb), gpu_ctx.alloc(m * hk * eb),
                              gpu_ctx.alloc(m * hk * eb))
    gpu_ctx.rope_half(q, dp, dc, ds, want_q, m, heads, d, table, True, io)
    gpu_ctx.rope_half(kk, dp, dc, ds, want_k, m, kv_heads, d, table, True, io)
    gpu_ctx.transpose_01(v, want_v, m, kv_heads, d, io)

    def part(lo, hi):
        return Int4Linear(hi - lo, k, packed[lo:hi], scales[lo:hi])
    fused = _stack_rows(_rope_pair_rows(part(0, hq), d), _rope_pair_rows(part(hq, hq + hk), d),
                        part(hq + hk, n))
    got_q, got_k, got_v = (gpu_ctx.zeros(m * hq * eb), gpu_ctx.zeros(m * hk * eb),
                           gpu_ctx.zeros(m * hk * eb))
    gpu_ctx.prefill_qkv(dx, gpu_ctx.upload(fused.packed), gpu_ctx.upload(fused.scales), dp, dc, ds,
                        got_q, got_k, got_v, m=m, heads=heads, kv_heads=kv_heads, depth=d, k=k,
                        group=group, table_rows=table, io_dtype=io, scale_dtype=ka.F16,
                        compute=compute)
    bits = np.uint32 if io == ka.F32 else np.uint16
    for got, want, planes in ((got_q, want_q, heads), (got_k, want_k, kv_heads),
                              (got_v, want_v, kv_heads)):
        a = got.download(io_np, (planes, m, d))
        b = want.download(io_np, (planes, m, d))
        assert np.array_equal(a.view(bits), b.view(bits))
    q_host = got_q.download(io_np, (heads, m, d))
    assert np.all(np.isnan(q_host[:, m // 2])) and not np.any(np.isnan(np.delete(q_host, m // 2, 1)))
    assert not np.any(np.isnan(got_v.download(io_np, (kv_heads, m, d))))


# ---- fp16 copies of the activations only a product reads (KRM_COMPUTE_F16 beside f32 io) ------

def test_fp16_activation_copies_give_the_bits_of_the_f32_activations(gpu_ctx):
    """KRM_COMPUTE_F16 rounds f32 activations to fp16 when a product reads them.  The producers
    can store that rounding themselves (krm_rms_norm_cast, KRM_CHUNK_OUT_F16, an fp16-io
    gate/up call) and the products read it through x_dtype: each piece equals the f32 route bit
    for bit."""
    rng = np.random.default_rng(77)
    m, k, n, group = 70, 512, 384, 128
    x = (rng.normal(size=(m, k)) * 3).astype(np.float32)
    w = rng.normal(size=k).astype(np.float32)
    dx, dw = gpu_ctx.upload(x), gpu_ctx.upload(w)
    # rms_norm: the cast form stores the f32 result rounded once
    n32, n16 = gpu_ctx.alloc(m * k * 4), gpu_ctx.alloc(m * k * 2)
    gpu_ctx.rms_norm(dx, dw, n32, m, k, 1e-5, ka.F32)
    gpu_ctx.rms_norm_cast(dx, dw, n16, m, k, 1e-5, ka.F32, ka.F16)
    normed = n32.download(np.float32, (m, k))
    assert np.array_equal(n16.download(np.float16, (m, k)).view(np.uint16),
                          normed.astype(np.float16).view(np.uint16))
    with pytest.raises(ka.GpuValidationError, match="f32 -> fp16"):
        gpu_ctx.rms_norm_cast(dx, dw, n16, m, k, 1e-5, ka.F16, ka.F32)
    # a product: f32 x under COMPUTE_F16 against the fp16 copy through x_dtype
    packed, _q, scale = helpers.synthetic_int4(rng, n, k, group)
    dpk, dsc = gpu_ctx.upload(packed), gpu_ctx.upload(scale)
    res = rng.normal(size=(m, n)).astype(np.float32)
    outs = []
    for xbuf, xd in ((n32, ka.F32), (n16, ka.F16)):
        out = gpu_ctx.upload(res)   # residual in place
        gpu_ctx.linear_i4_rows(xbuf, dpk, dsc, out, m, n, k, group, residual=out,
                               io_dtype=ka.F32, scale_dtype=ka.dtype_code(scale.dtype),
                               compute=ka.COMPUTE_F16, x_dtype=xd)
        outs.append(out.download(np.float32, (m, n)))
    assert np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    want = oracle.linear_i4(normed.astype(np.float16).astype(np.float32), packed,
                            np.asarray(scale, np.float32), np.zeros(n, np.float32), n, k, group) + res
    assert np.allclose(outs[1], want, rtol=1e-5, atol=2e-4)
    # gate/up: fp16 in and out equals the f32 route's result rounded once
    act32, act16 = gpu_ctx.alloc(m * (n // 2) * 4), gpu_ctx.alloc(m * (n // 2) * 2)
    gpu_ctx.linear_i4_rows(n32, dpk, dsc, act32, m, n, k, group, io_dtype=ka.F32,
                           scale_dtype=ka.dtype_code(scale.dtype), compute=ka.COMPUTE_F16,
                           epilogue=ka.EPILOGUE_SILU_PAIRS)
    gpu_ctx.linear_i4_rows(n16, dpk, dsc, act16, m, n, k, group, io_dtype=ka.F16,
                           scale_dtype=ka.dtype_code(scale.dtype), compute=ka.COMPUTE_F16,
                           epilogue=ka.EPILOGUE_SILU_PAIRS)
    assert np.array_equal(act16.download(np.float16, (m, n // 2)).view(np.uint16),
                          act32.download(np.float32, (m, n // 2)).astype(np.float16).view(np.uint16))
    # the combinations the kernel does not have are rejected
    with pytest.raises(ka.GpuValidationError, match="x_dtype"):
        gpu_ctx.linear_i4_rows(n16, dpk, dsc, act32, m, n, k, group, io_dtype=ka.F32,
                               scale_dtype=ka.dtype_code(scale.dtype), compute=ka.COMPUTE_F32,
                               x_dtype=ka.F16)
    with pytest.raises(ka.GpuValidationError, match="x_dtype"):
        gpu_ctx.linear_i4_rows(n32, dpk, dsc, act16, m, n, k, group, io_dtype=ka.F16,
                               scale_dtype=ka.dtype_code(scale.dtype), compute=ka.COMPUTE_F16,
                               x_dtype=ka.F32)


def test_attention_chunk_fp16_output_is_the_f32_output_rounded(gpu_ctx):
    rng = np.random.default_rng(5)
    heads, kvh, m, d, cap, past, query = 8, 2, 40, 64, 128, 50, 37
    q = gpu_ctx.upload(rng.normal(size=(heads, m, d)).astype(np.float32))
    ik = gpu_ctx.upload(rng.normal(size=(kvh, m, d)).astype(np.float32))
    iv = gpu_ctx.upload(rng.normal(size=(kvh, m, d)).astype(np.float32))
    sk = gpu_ctx.upload(rng.normal(size=(kvh, cap, d)).astype(np.float32))
    sv = gpu_ctx.upload(rng.normal(size=(kvh, cap, d)).astype(np.float32))
    o32 = gpu_ctx.upload(np.full(m * heads * d, 7.0, np.float32))
    o16 = gpu_ctx.upload(np.full(m * heads * d, 7.0, np.float16))
    spec = dict(batch=1, heads=heads, kv_heads=kvh, chunk_rows=m, depth=d, capacity=cap, window=0,
                half_scale=oracle.half_scale(d), past=past, query=query, row_major=True)
    gpu_ctx.attention_chunk(q, ik, iv, sk, sv, o32, **spec)
    gpu_ctx.attention_chunk(q, ik, iv, sk, sv, o16, out_f16=True, **spec)
    a = o32.download(np.float32, (m, heads, d))
    b = o16.download(np.float16, (m, heads, d))
    assert np.array_equal(b.view(np.uint16), a.astype(np.float16).view(np.uint16))
    assert np.all(b[query:] == 0) and np.any(b[:query] != 0)


def test_prefill_with_fp16_activation_copies_equals_prefill_without(gpu_ctx):
    """A whole chunk through the decoder under KRM_COMPUTE_F16: logits and the appended state are
    the same bits with and without the fp16 copies."""
    config = LlamaConfig(layers=2, d_model=256, ffn=384, heads=4, kv_heads=2, head_dim=64,
                         vocab=512, group_size=128, max_position=64)
    weights = random_weights(config, seed=6)
    rng = np.random.default_rng(2)
    ids = rng.integers(0, config.vocab, size=(1, 40)).astype(np.int32)
    pos = np.arange(40, dtype=np.int32).reshape(1, 40)
    results = []
    for copies in (True, False):
        session = LlamaDecoderSession(gpu_ctx, weights, io_dtype=ka.F32, kv_dtype=ka.F32,
                                      chunk_length=40, prefill_compute=ka.COMPUTE_F16)
        session.half_activations = copies
        ctx = session.create_generation_context(capacity=64, chunk_length=40)
        token, logits = session.run(ids, pos, 36, context=ctx, query_length=37, want_logits=True)
        state = ctx.slots_k[1].download(np.float32, (2, 64, 64))[:, :37].copy()
        results.append((token.copy(), logits.copy(), state))
        ctx.dispose()
        session.close()
    assert np.array_equal(results[0][1].view(np.uint32), results[1][1].view(np.uint32))
    assert np.array_equal(results[0][2].view(np.uint32), results[1][2].view(np.uint32))
    assert np.array_equal(results[0][0], results[1][0])


# ---- layers that differ: sliding windows, head dims per layer kind, KV-sharing layers ----------
# (tools/export-recipes/gemma4/export_decode.py:59-82,510-527).  Sliding layers: head dim 64,
# window 8 (the sequence passes it, so the band and the ring both matter); full layers: head
# dim 128 here, 32 in the second config (the attention's generic kernel); layers 3 and 4 read
# the K / V rows and slots of layers 1 and 2.
MIXED = LlamaConfig(layers=5, d_model=256, ffn=384, heads=8, kv_heads=2, head_dim=64, vocab=512,
                    group_size=128, max_position=64,
                    layer_windows=(8, 8, 0, 8, 0), layer_head_dims=(64, 64, 128, 64, 128),
                    layer_kv_source=(0, 1, 2, 1, 2))
MIXED_SMALL_DIMS = LlamaConfig(layers=4, d_model=256, ffn=384, heads=8, kv_heads=4, head_dim=32,
                               vocab=512, group_size=128, max_position=64,
                               layer_windows=(0, 12, 0, 12), layer_head_dims=(32, 16, 32, 16),
                               layer_kv_source=(0, 1, 0, 1))


# head dims 256 (sliding, shared by layer 2) and 64: the sizes of a Gemma-4 sliding layer
MIXED_256 = LlamaConfig(layers=3, d_model=256, ffn=384, heads=4, kv_heads=1, head_dim=256,
                        vocab=512, group_size=128, max_position=64,
                        layer_windows=(8, 0, 8), layer_head_dims=(256, 64, 256),
                        layer_kv_source=(0, 1, 0))


@pytest.mark.parametrize("config,chunk", [(MIXED, 8), (MIXED, 32), (MIXED_SMALL_DIMS, 8),
                                          (MIXED_SMALL_DIMS, 24), (MIXED_256, 8), (MIXED_256, 32)],
                         ids=["chunks of 8", "chunks of 32 (few-row launches)",
                              "small dims, chunks of 8", "small dims, chunks of 24",
                              "head dim 256, chunks of 8", "head dim 256, chunks of 32"])
def test_layers_that_differ_match_the_full_reforward(gpu_ctx, config, chunk):
    """Session over a decoder whose layers differ against the oracle's full re-forward with the
    explicit band mask (no state slots, no ring): prefill in chunks (the last one padded), then
    one-row steps, teacher-forced; every run's last-row logits within atol 2e-4 (the gate of the
    uniform chain test).  The sequence is longer than the windows, so sliding layers wrap their
    rings; sharing layers must see their owner's rows of this step and its slots before the
    append."""
    weights = random_weights(config, seed=31)
    total, prompt_len = 44, 29
    ids = np.random.default_rng(17).integers(0, config.vocab, size=total).astype(np.int32)
    want = helpers.oracle_decoder_logits(weights, ids)
    session = LlamaDecoderSession(gpu_ctx, weights, chunk_length=chunk)
    ctx = session.create_generation_context(capacity=64, chunk_length=chunk)
    assert [ctx.layer_capacity[li] for li in range(config.layers)] == \
        [config.window_of(li) or 64 for li in range(config.layers)]
    worst = 0.0
    for piece in plan_prefill_chunks(prompt_len, chunk):
        n = piece.query_length
        cid = np.zeros((1, chunk), dtype=np.int32)
        cpos = np.zeros((1, chunk), dtype=np.int32)
        cid[0, :n] = ids[piece.position:piece.position + n]
        cpos[0, :n] = np.arange(piece.position, piece.position + n)
        _tok, logits = session.run(cid, cpos, n - 1, context=ctx, query_length=n,
                                   want_logits=True)
        worst = max(worst, float(np.max(np.abs(logits[0] - want[piece.position + n - 1]))))
    for pos in range(prompt_len, total):
        token, logits = session.run(ids[pos:pos + 1][None], np.array([[pos]], dtype=np.int32), 0,
                                    context=ctx, query_length=1, want_logits=True)
        worst = max(worst, float(np.max(np.abs(logits[0] - want[pos]))))
        top = np.sort(want[pos])
        if top[-1] - top[-2] > 4e-4:
            assert int(token[0, 0, 0]) == int(np.argmax(want[pos])), pos
    assert ctx.past == total
    assert worst <= 2e-4, worst
    with pytest.raises(ka.ExecutionError, match="sliding"):
        ctx.rewind(3)
    ctx.dispose()
    session.close()


def test_layers_that_differ_replayed_decode_and_file_session(gpu_ctx):
    """The recorded step of a decoder whose layers differ replays to the step-by-step tokens,
    and a session built from the model file gives the session from arrays bit for bit."""
    from model_file import decoder_model_file
    weights = random_weights(MIXED, seed=32)
    from karume_amd.decoder import DecoderWeights
    loaded = DecoderWeights.from_model(ka.open_model(decoder_model_file(weights)))
    assert loaded.config == MIXED
    prompt = [int(t) for t in np.random.default_rng(5).integers(0, MIXED.vocab, size=13)]
    new = 20
    results = []
    for w in (weights, loaded):
        session = LlamaDecoderSession(gpu_ctx, w, chunk_length=8)
        stepwise = generate_greedy(session, prompt=prompt, max_new_tokens=new, chunk_length=8,
                                   max_position=MIXED.max_position)
        ctx = session.create_generation_context(capacity=MIXED.max_position, chunk_length=8)
        token = None
        for piece in plan_prefill_chunks(len(prompt), 8):
            n = piece.query_length
            cid = np.zeros((1, 8), dtype=np.int32)
            cpos = np.zeros((1, 8), dtype=np.int32)
            cid[0, :n] = prompt[piece.position:piece.position + n]
            cpos[0, :n] = np.arange(piece.position, piece.position + n)
            token, logits = session.run(cid, cpos, n - 1, context=ctx, query_length=n,
                                        want_logits=True)
        first = int(token[0, 0, 0])
        replayed = [first] + session.decode_tokens(ctx, first, new - 1)
        assert replayed == stepwise
        assert ctx.past == len(prompt) + new - 1
        ctx.dispose()
        session.close()
        results.append((stepwise, logits.tobytes()))
    assert results[0] == results[1]
