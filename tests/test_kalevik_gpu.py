"""The Kalevik decoder on the GPU against the plain implementation (tests/plain_kalevik.py): every mechanism alone
through its kernels, then the engine whole, token by token, in portions down to two tokens, in mixed batches on reused
pages and slots, long decoding, and greedy generation through the scheduler. The configurations are made here
(tests/kalevik_tiny.py) and differ from each other in every size."""
import io
import math
import os

import numpy as np
import pytest
import torch

import plain_kalevik as plain
from kalevik_tiny import CONFIGS, STDS, make_kalevik_folder, without_choice
from replay_tools import collect, mixed, portions, prefill_then_decode, round_up, to_lines, whole

pytestmark = pytest.mark.gpu

F32_BOUND = 2e-5        # of the logits' scale: float32 against float64, sums in other orders
BF16_BOUND = 0.06       # of the logits' scale: what the format costs on these models; a fault costs far more
ROUTER_MARGIN = 0.01    # a token whose choice of experts hangs on less than this may choose otherwise in bfloat16
F = torch.float64
_models = {}


def model_for(tmp_path_factory, which, dtype="float32"):
    """The model ``which``; for a bfloat16 engine the same model with every token sent through all experts
    (``kalevik_tiny.without_choice`` says why)."""
    choice = dtype == "float32"
    if (which, choice) not in _models:
        folder = make_kalevik_folder(tmp_path_factory.mktemp(f"kalevik_{which}"), which, choice)
        _models[(which, choice)] = (folder, plain.read_config(folder), plain.read_tensors(folder))
    return _models[(which, choice)]


def tokens_for(seed, count, vocab):
    return np.random.default_rng(seed).integers(0, vocab, size=count).tolist()


def row_errors(got, want):
    difference = got - want
    difference = difference - difference.mean(-1, keepdims=True)
    return np.sqrt((difference ** 2).mean(-1)) / np.sqrt(((want - want.mean(-1, keepdims=True)) ** 2).mean())


def run_trace(folder, dtype, steps, out_dir, max_tokens, max_requests=4, **options):
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype=dtype, max_tokens=max_tokens, max_requests=max_requests, **options)
    report = io.StringIO()
    replay(engine, io.StringIO(to_lines(steps)), str(out_dir), report)
    assert report.getvalue().split() == [word for step in steps for word in ("done", str(step["step"]))]
    engine.cache.check()
    assert not engine.cache.requests and all(free == group.pool.num_pages for free, group in zip(engine.cache.free_pages(), engine.cache.groups))
    return engine


_plain_runs = {}


def plain_run(config, weights, tokens):
    """Logits, the residual stream after every layer run, every position's smallest router margin, and every position's
    sensitivity: how far the plain implementation itself, run in 32-bit, lies from its 64-bit run there, over twice its
    median (at least 1). A sublayer's result is divided by its own root mean square before it joins the stream, and so is
    every head of a retention; where such a result nearly cancels, any format's error is divided by the same small
    number, in the plain run as in the engine."""
    key = (id(weights), tuple(tokens))
    if key not in _plain_runs:
        streams, margins = [], []
        logits = plain.forward(config, weights, tokens, layers_out=streams, margins=margins).numpy()
        margin = np.asarray(margins).reshape(-1, len(tokens)).min(0) if margins else np.full(len(tokens), np.inf)
        plain.F = torch.float32
        try:
            single = row_errors(plain.forward(config, weights, tokens).double().numpy(), logits)
        finally:
            plain.F = torch.float64
        sensitivity = np.maximum(1.0, single / (2.0 * np.median(single)))
        _plain_runs[key] = (logits, torch.stack(streams).numpy(), margin, sensitivity)
    return _plain_runs[key]


def plain_logits(config, weights, tokens):
    return plain_run(config, weights, tokens)[0]


def within_bound(errors, dtype):
    """``errors`` are already divided by their positions' sensitivity (``plain_run``). Float32: every position within the
    bound. bfloat16: a token that went to another expert than in the plain run (left out itself) also moves what later
    positions read from the cache and the state: nine in ten positions are held to the bound and none may be off by
    three times as much. What a fault of a kernel does (a chunk off by one, a lost state, a wrong page) shows in
    float32, where every position is held, and costs far more than this in either format."""
    if dtype == "float32" or len(errors) < 10:
        return errors.max() < (F32_BOUND if dtype == "float32" else 2 * BF16_BOUND)
    return np.quantile(errors, 0.9) < BF16_BOUND and errors.max() < 3 * BF16_BOUND


def check_against_plain(steps, out_dir, requests, config, weights, dtype):
    got = collect(steps, str(out_dir), config["vocab"])
    for rid, tokens in requests.items():
        want, _, margin, sensitivity = plain_run(config, weights, tokens)
        places = sorted(place for (request, place) in got if request == rid)
        assert places, f"no logits came back for {rid}"
        errors = row_errors(np.stack([got[(rid, place)] for place in places]), want[places]) / sensitivity[places]
        if dtype != "float32":
            errors = np.where(margin[places] >= ROUTER_MARGIN, errors, 0.0)
        assert within_bound(errors, dtype), f"{rid}: position {places[int(errors.argmax())]} is off by {errors.max():.3g} of the scale"


def device(array, dtype=torch.float32):
    return torch.as_tensor(np.asarray(array), dtype=dtype).cuda().contiguous()


def as_bf16(array):
    return torch.as_tensor(np.asarray(array), dtype=torch.float32).to(torch.bfloat16).to(torch.float64).numpy()


def t64(array):
    return torch.as_tensor(np.asarray(array), dtype=F)


# ---- mechanisms alone -------------------------------------------------------------------------------------------
def test_embedding_times_a_factor():
    from microllm_rocm_amd.ops import kernels
    table = as_bf16(np.random.default_rng(0).normal(size=(11, 37)))
    ids = [3, 0, 10, 3]
    for scale in (1.0, 3.0, 0.37):
        got = kernels.embedding(device(table, torch.bfloat16), device(ids, torch.int32), scale=scale).cpu().numpy()
        assert np.abs(got - table[ids] * scale).max() < 1e-6 * max(scale, 1.0)


@pytest.mark.parametrize("width", [64, 50, 7, 1000])
def test_rows_that_join_the_stream_with_a_normed_delta(width):
    """``h + norm(delta) * w_after + rows`` in one kernel with the norm that reads the stream next: what a pass of a
    looped range begins with."""
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(width)
    h, delta, rows = rng.normal(size=(6, width)) * 3, rng.normal(size=(6, width)) * 5, rng.normal(size=(6, width)) * 2
    after, weight = rng.normal(size=width) + 1, rng.normal(size=width) + 1
    joined = t64(h) + plain.rms(t64(delta), 1e-5) * t64(after) + t64(rows)
    want = (plain.rms(joined, 1e-5) * t64(weight)).numpy()
    stream = device(h)
    got = kernels.rms_norm_after(stream, device(delta), device(after), 1e-5, 1.0, device(weight), 1e-5, torch.float32, write_h=True,
                                 extra=device(rows))
    assert np.abs(got.cpu().numpy() - want).max() < 2e-5 and np.abs(stream.cpu().numpy() - joined.numpy()).max() < 2e-5
    chosen = device([4, 1], torch.int32)
    got = kernels.rms_norm_after(device(h), device(delta), device(after), 1e-5, 1.0, device(weight), 1e-5, torch.float32, rows=chosen,
                                 extra=device(rows))
    assert np.abs(got.cpu().numpy() - want[[4, 1]]).max() < 2e-5


def test_rows_join_the_stream_whatever_the_layer_before_left():
    """``Model`` adds the embedding's rows before an entry that asks for them: along with a delta that is still to be
    normed, or at once where the delta is plain (another arrangement) or there is none."""
    from microllm_rocm_amd.parts.model import Model
    from microllm_rocm_amd.parts.norm import NormedDelta
    rng = np.random.default_rng(9)
    h, delta, rows = (rng.normal(size=(5, 24)) for _ in range(3))
    stream = device(h)
    assert Model._add_to_stream(stream, None, device(rows)) is None
    assert np.abs(stream.cpu().numpy() - (h + rows)).max() < 1e-6
    stream = device(h)
    assert Model._add_to_stream(stream, device(delta), device(rows)) is None
    assert np.abs(stream.cpu().numpy() - (h + delta + rows)).max() < 1e-6
    stream, parts = device(h), device(np.stack([delta * 0.25, delta * 0.75]))
    assert Model._add_to_stream(stream, parts, device(rows)) is None
    assert np.abs(stream.cpu().numpy() - (h + delta + rows)).max() < 1e-6
    stream = device(h)
    normed = NormedDelta(device(delta), device(np.ones(24)), 1e-5, 1.0)
    taken = Model._add_to_stream(stream, normed, device(rows))
    assert isinstance(taken, NormedDelta) and taken.extra is not None and normed.extra is None
    assert np.array_equal(stream.cpu().numpy(), device(h).cpu().numpy())       # nothing added yet: the next norm's kernel does it
    want = t64(rows) + plain.rms(t64(delta), 1e-5)
    assert np.abs(taken.resolved().cpu().numpy() - want.numpy()).max() < 1e-5
    with pytest.raises(ValueError):
        taken.with_extra(device(rows))


def test_activations_by_name():
    from microllm_rocm_amd.ops import kernels
    z = np.random.default_rng(2).normal(size=(5, 33)) * 3
    wants = {"silu": plain.silu(t64(z)), "gelu_erf": plain.gelu_erf(t64(z)),
             "gelu_tanh": 0.5 * t64(z) * (1 + torch.tanh(math.sqrt(2 / math.pi) * (t64(z) + 0.044715 * t64(z) ** 3)))}
    for kind, want in wants.items():
        assert np.abs(kernels.activation(device(z), kind, torch.float32).cpu().numpy() - want.numpy()).max() < 1e-5, kind
        parts = np.stack([z * 0.25, z * 0.5, z * 0.25])
        assert np.abs(kernels.activation(device(parts), kind, torch.float32).cpu().numpy() - want.numpy()).max() < 1e-5, kind
        rounded = kernels.activation(device(z), kind, torch.bfloat16).float().cpu().numpy()
        assert np.abs(rounded - want.numpy()).max() < 0.01 * np.abs(want.numpy()).max(), kind
    assert abs(float(plain.gelu_erf(t64([1.0]))[0]) - 0.8413447460685429) < 1e-12        # the exact form, not the tanh one (0.84119)


def chunked(q, k, v, gate, scale, chunk, portions_of, mfma, norm_weights=None, rot=None, eps=1e-5, page_size=16):
    """The engine's kernels on one request: the norm of queries and keys, their rotation, keys and values into pages
    that are scattered and out of order, and the attention inside chunks with one added to the softmax's denominator and
    a gate a head, in the given portions: plain pages and the kernel that takes a wave a token and head (float32), or the
    tiled pages and the MFMA kernels (bfloat16). ``rot``: (base, dims, factor)."""
    from types import SimpleNamespace
    from microllm_rocm_amd.cache.layout import key_page_shape, value_page_shape
    from microllm_rocm_amd.ops import kernels
    from microllm_rocm_amd.parts.attention import QueryTilePlanner
    n, heads, dim = q.shape
    kv_heads, vdim = k.shape[1], v.shape[2]
    dtype = torch.bfloat16 if mfma else torch.float32
    blocks = -(-n // page_size)
    pages = [2 + 3 * block for block in reversed(range(blocks))]
    count = 3 * blocks + 2
    table = device([pages], torch.int32)
    sink = torch.zeros(heads, device="cuda")
    q_weight = k_weight = None
    if norm_weights is not None:
        q_weight, k_weight = device(norm_weights[0]), device(norm_weights[1])
    inv_freq = None
    if rot is not None:
        base, dims, factor = rot
        inv_freq = device(base ** (-2.0 * np.arange(dims // 2) / dims) / factor, torch.float64)
    if mfma:
        k_pages = torch.zeros(key_page_shape(count, kv_heads, page_size, dim), dtype=dtype, device="cuda")
        v_pages = torch.zeros(value_page_shape(count, kv_heads, page_size, dim), dtype=dtype, device="cuda")
        planner = QueryTilePlanner(True)
    else:
        k_pages = torch.full((count, page_size, kv_heads, dim), 1e4, dtype=dtype, device="cuda")      # what is not this request's must not count
        v_pages = torch.full((count, page_size, kv_heads, vdim), 1e4, dtype=dtype, device="cuda")
    out, first = [], 0
    for portion in portions_of:
        portion = min(portion, n - first)
        if portion <= 0:
            break
        rows = slice(first, first + portion)
        qkv = np.concatenate([q[rows].reshape(portion, -1), k[rows].reshape(portion, -1), v[rows].reshape(portion, -1), gate[rows]], axis=1)
        positions = np.arange(first, first + portion)
        slots = [pages[p // page_size] * page_size + p % page_size for p in positions]
        pos, seq_of_token = device(positions, torch.int32), device(np.zeros(portion), torch.int32)
        proj = device(qkv)
        queries = kernels.qk_norm_store(proj, q_weight, k_weight, eps, pos, device(slots, torch.int32), 0.0, 1, k_pages, v_pages, heads,
                                        kv_heads, dim, vdim, dtype, tiled_page_size=page_size if mfma else 0, normed=norm_weights is not None,
                                        cos_sin=kernels.rope_table(pos, inv_freq) if inv_freq is not None else None, further_columns=heads)
        gates = proj[:, proj.shape[1] - heads:]
        if mfma:
            host = SimpleNamespace(counts=[portion], cu=np.array([0, portion]), starts=[first], totals=[first + portion],
                                   single_tokens_only=portion == 1, n_tokens=portion, n_seqs=1, page_size=page_size)
            ctx = SimpleNamespace(max_count=portion, planned_total=first + portion, max_total=first + portion, n_tokens=portion,
                                  seq_of_token=seq_of_token, positions=pos, fixed=False, host=host, tokens=pos, planned={})
            arrays, values = planner.plan(host)
            plan = SimpleNamespace(**values, **{name: device(array, torch.int32) for name, array in arrays.items()})
            ctx.plan_of = lambda _planner: plan
            view = SimpleNamespace(block_table=table, page_size=page_size)
            found = torch.empty((portion, heads * dim), dtype=dtype, device="cuda")
            extras = kernels.AttentionExtras(None, sink, 1.0, chunk=chunk, gate=gates)
            kernels.paged_attention(queries, k_pages, v_pages, view, ctx, scale, 0, heads, kv_heads, dim, planner=planner, extras=extras, out=found)
        else:
            found = kernels.bias_attention(queries, k_pages, v_pages, table, seq_of_token, pos, None, sink, scale, 1.0, heads, kv_heads, dim,
                                           vdim, chunk=chunk, gate=gates)
        out.append(found.float().cpu().numpy().reshape(portion, heads, vdim))
        first += portion
    return np.concatenate(out)


def plain_chunked(q, k, v, gate, scale, chunk, norm_weights=None, rot=None, eps=1e-5):
    q, k = t64(q), t64(k)
    if norm_weights is not None:
        q, k = plain.rms(q, eps) * t64(norm_weights[0]), plain.rms(k, eps) * t64(norm_weights[1])
    if rot is not None:
        positions = torch.arange(q.shape[0])
        q, k = plain.turn_halves(q, positions, rot[0], rot[1], rot[2]), plain.turn_halves(k, positions, rot[0], rot[1], rot[2])
    return (plain.attend_in_chunks(q, k, t64(v), scale, chunk) * torch.sigmoid(t64(gate))[:, :, None]).numpy()


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,chunk,rot,n,mfma", [
    (4, 2, 24, 16, 19, (100.0, 8, 2.0), 70, False), (3, 1, 10, 6, 1, (77.0, 10, 1.0), 33, False), (5, 5, 6, 11, 1000, None, 130, False),
    (1, 1, 128, 200, 64, (1e4, 64, 4.0), 150, False), (6, 2, 16, 16, 19, (100.0, 8, 2.0), 150, True), (8, 2, 32, 32, 32, (5e5, 32, 1.0), 300, True),
    (2, 1, 48, 48, 65, (1e4, 16, 8.0), 270, True), (4, 4, 96, 96, 130, None, 300, True), (1, 1, 128, 128, 1, (1e4, 128, 1.0), 70, True),
    (3, 3, 64, 64, 1000, (1e4, 32, 4.0), 280, True)])
def test_attention_inside_chunks(heads, kv_heads, dim, vdim, chunk, rot, n, mfma):
    """Random queries, keys, values and gates with a norm of queries and keys and a rotation of part of the head; whole,
    decoded, in portions of two and of sizes that cut pages and chunks anywhere."""
    rng = np.random.default_rng(dim + chunk)
    q, k, v = (as_bf16(rng.normal(size=shape)) for shape in ((n, heads, dim), (n, kv_heads, dim), (n, kv_heads, vdim)))
    gate = as_bf16(rng.normal(size=(n, heads)) * 2)
    weights = (rng.normal(size=dim) + 1, rng.normal(size=dim) + 1)
    want = plain_chunked(q, k, v, gate, 0.3, chunk, weights, rot)
    bound = 0.03 * np.abs(want).max() if mfma else 2e-5
    got = chunked(q, k, v, gate, 0.3, chunk, [n], mfma, weights, rot)
    assert np.abs(got - want).max() < bound
    for portions_of in ([max(n - 40, 2)] + [1] * 40, [2] * (n // 2 + 1), [1] * 5 + [3, 16, 1, 2, 31, 129, 1, 1, 500]):
        again = chunked(q, k, v, gate, 0.3, chunk, portions_of, mfma, weights, rot)
        assert np.abs(again - want).max() < bound, portions_of
        if not mfma:
            assert np.array_equal(again, got), portions_of      # a row does not depend on how the request was cut


@pytest.mark.parametrize("mfma", [False, True])
def test_the_added_one_in_the_denominator(mfma):
    """All scores are zero: a query that sees ``m`` keys weighs each ``1 / (m + 1)``, so the first token of every chunk
    returns half of its own value; an open gate (a large number) lets that through whole, a gate of 0 halves it again."""
    heads, n, chunk, dim = 2, 50, 7, 16
    q, k = np.zeros((n, heads, dim)), np.zeros((n, 1, dim))
    v = as_bf16(np.random.default_rng(0).normal(size=(n, 1, dim)))
    gate = np.stack([np.full(n, 30.0), np.zeros(n)], axis=1)
    got = chunked(q, k, v, gate, 1.0, chunk, [n - 9] + [1] * 9, mfma)
    for query in (0, 6, 7, 13, 14, 41, 42, 48, 49):
        first = query // chunk * chunk
        want = v[first:query + 1, 0].sum(0) / (query - first + 2)
        assert np.abs(got[query, 0] - want).max() < (0.02 if mfma else 1e-5), query
        assert np.abs(got[query, 1] - want / 2).max() < (0.02 if mfma else 1e-5), query


@pytest.mark.parametrize("mfma", [False, True])
@pytest.mark.parametrize("chunk", [1, 2, 15, 16, 17, 64, 65, 130, 1000])
def test_chunk_edges_far_keys_and_first_tokens(mfma, chunk):
    """One key's score is made to stand out (the query and that key alone point along one channel, far above every other
    score and above the added one): the first key of the query's chunk takes all the weight, the last key of the chunk
    before takes none, wherever the edge falls in a page or a tile of keys; in a prompt, decoded, and in portions of two."""
    rng = np.random.default_rng(chunk)
    n, heads, dim = 300, 2, 16
    q = as_bf16(rng.normal(size=(n, heads, dim)) * 0.1)
    k, v = as_bf16(rng.normal(size=(n, 1, dim)) * 0.1), as_bf16(rng.normal(size=(n, 1, dim)))
    k[:, 0, 3] = 0.0
    gate = np.full((n, heads), 30.0)
    bound = 0.02 if mfma else 1e-4
    for query in (n - 1, 200, 128, 64, 16):
        first = query // chunk * chunk
        for key in sorted({first, first - 1, query, query - 1, 0}):      # the oldest key still seen, the newest no longer seen, itself, the one before, the first token
            if key < 0:
                continue
            sharp_q, sharp_k = q.copy(), k.copy()
            sharp_q[query, 0] = 0.0
            sharp_q[query, 0, 3] = 5.0
            sharp_k[key, 0] = 0.0
            sharp_k[key, 0, 3] = 5.0
            want = plain_chunked(sharp_q, sharp_k, v, gate, 2.0, chunk)       # the standing-out score is 50
            seen = key >= first
            assert (np.abs(want[query, 0] - v[key, 0]).max() < 1e-6) == seen      # the plain run itself shows the edge
            pairs = min(70 if query == 128 else 8, (query + 1) // 2)
            in_twos = ([query + 1 - 2 * pairs] if query + 1 > 2 * pairs else []) + [2] * pairs
            for portions_of in ([query + 1], [query, 1], in_twos):       # a prompt's last token, decoded alone, the second of a portion of two
                got = chunked(sharp_q[:query + 1], sharp_k[:query + 1], v[:query + 1], gate[:query + 1], 2.0, chunk, portions_of, mfma)
                assert np.abs(got[query, 0] - want[query, 0]).max() < bound, (query, key, portions_of)


def retained(q, k, v, gate, decay, portions_of, eps=1e-5, out_scale=1.0, long_portions=None):
    """The retention's kernels on one request in the given portions: the walk with one decay a head, then every head's
    result divided by its root mean square and multiplied by ``silu(gate)``; the state carried in a slot."""
    from microllm_rocm_amd.ops import kernels
    n, heads, dim = q.shape
    vdim = v.shape[2]
    keys, values = heads * dim, heads * vdim
    state = torch.zeros((3, heads, dim, vdim), device="cuda")
    state[0] = state[2] = 1e4       # other requests' slots
    decay_row = device(np.repeat(np.asarray(decay, dtype=np.float64), dim))
    out, first = [], 0
    for portion in portions_of:
        portion = min(portion, n - first)
        if portion <= 0:
            break
        rows = slice(first, first + portion)
        proj = device(np.concatenate([q[rows].reshape(portion, -1), k[rows].reshape(portion, -1), v[rows].reshape(portion, -1),
                                      gate[rows].reshape(portion, -1)], axis=1))
        walked = kernels.gla_scan(proj, 0, keys, 2 * keys, decay_row, state, device([0, portion], torch.int32), device([1], torch.int32), 1,
                                  heads, dim, vdim, dim ** -0.5, long_portions=portion >= 8 if long_portions is None else long_portions)
        out.append(kernels.gla_gate(walked, proj, 2 * keys + values, None, eps, heads, vdim, out_scale, torch.float32).cpu().numpy())
        first += portion
    assert float(state[0].min()) == 1e4 and float(state[2].max()) == 1e4
    return np.concatenate(out).reshape(n, heads, vdim)


@pytest.mark.parametrize("heads,dim,vdim,n", [(3, 12, 10, 70), (1, 9, 14, 40), (4, 8, 8, 90), (2, 40, 7, 50), (1, 128, 12, 35), (6, 32, 32, 300)])
def test_retention_with_one_decay_a_head(heads, dim, vdim, n):
    rng = np.random.default_rng(heads * dim)
    q, k, v, gate = (rng.normal(size=shape) for shape in ((n, heads, dim), (n, heads, dim), (n, heads, vdim), (n, heads, vdim)))
    decay = [1.0, 0.0, 0.7, 0.97, 0.998046875, 0.5][:heads]
    walked = plain.retain(t64(q), t64(k) * dim ** -0.5, t64(v), decay)
    want = (plain.rms(walked, 1e-5) * plain.silu(t64(gate))).numpy()
    got = retained(q, k, v, gate, decay, [n])
    assert np.abs(got - want).max() < 3e-5 * max(1.0, np.abs(want).max())
    for portions_of in ([max(n - 30, 2)] + [1] * 30, [2] * (n // 2 + 1), [1] * 5 + [3, 16, 1, 2, 31, 129, 1, 1, 500]):
        again = retained(q, k, v, gate, decay, portions_of)
        assert np.array_equal(again, got), portions_of          # the state carried over a cut is the state walked through it
    assert np.array_equal(retained(q, k, v, gate, decay, [n], long_portions=False), got)
    if heads > 1:       # a decay of zero keeps the token alone: o = (k . q) v before the norm
        alone = (t64(k[:, 1]) * dim ** -0.5 * t64(q[:, 1])).sum(-1, keepdim=True) * t64(v[:, 1])
        assert torch.allclose(walked[:, 1], alone, atol=1e-12)


def test_a_far_token_stays_in_the_state():
    """A decay of one forgets nothing: the first token's value, written along one key channel that no later key touches,
    is read back whole by the last query 400 tokens on; with a decay of 1/2 nothing of it is left."""
    n, dim, vdim = 401, 16, 8
    rng = np.random.default_rng(5)
    q, k = np.zeros((n, 2, dim)), rng.normal(size=(n, 2, dim))
    v, gate = rng.normal(size=(n, 2, vdim)), np.full((n, 2, vdim), 30.0)
    k[:, :, 3] = 0.0
    k[0, :, 3] = 4.0
    q[n - 1, :, 3] = 1.0
    for portions_of in ([n], [n - 1, 1], [100, 2, 2, 297]):
        got = retained(q, k, v, gate, [1.0, 0.5], portions_of)
        want = v[0, 0] / math.sqrt((v[0, 0] ** 2).mean() + 1e-5 / (4.0 * dim ** -0.5) ** 2) * 30.0      # silu(30) = 30
        assert np.abs(got[n - 1, 0] - want).max() < 3e-3, portions_of
        assert np.abs(got[n - 1, 1]).max() < 1e-20 / 1e-5 ** 0.5, portions_of


@pytest.mark.parametrize("experts,top,groups,keep", [(8, 2, 4, 2), (12, 4, 4, 3), (6, 1, 3, 1), (16, 4, 4, 4), (5, 3, 0, 0), (12, 3, 6, 2), (64, 6, 8, 3), (100, 6, 10, 4), (300, 8, 0, 0)])
def test_choice_of_experts_among_the_best_groups(experts, top, groups, keep):
    from microllm_rocm_amd.ops import kernels
    rng = np.random.default_rng(experts + top)
    z = rng.normal(size=(200, experts + 1)) * 2
    ids, weights, shared = kernels.moe_route(device(z), experts, top, softmax_scores=True, renormalize=False, shared_at=experts,
                                             groups=groups, keep=keep)
    scores = torch.softmax(t64(np.asarray(device(z).cpu())[:, :experts]), dim=-1)
    for token in range(z.shape[0]):
        want = plain.route(scores[token], top, groups or 1, keep or 1)
        assert ids[token].tolist() == want, token
        assert np.abs(weights[token].cpu().numpy() - scores[token, want].numpy()).max() < 1e-6
    assert np.abs(shared.cpu().numpy() - 1 / (1 + np.exp(-z[:, experts]))).max() < 1e-6


@pytest.mark.parametrize("dtype,grouped", [(torch.float32, False), (torch.bfloat16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("width,ff,experts,top,n", [(64, 24, 8, 2, 50), (50, 20, 6, 1, 9), (96, 64, 16, 4, 200), (40, 7, 3, 3, 5)])
def test_experts_of_one_inner_weight_and_the_exact_gelu(dtype, grouped, width, ff, experts, top, n):
    from microllm_rocm_amd.ops import kernels
    if grouped and (width % 8 or ff % 8):
        pytest.skip("the tiled products take widths in steps of 8")
    rng = np.random.default_rng(width + ff)
    x, up, down = as_bf16(rng.normal(size=(n, width))), as_bf16(rng.normal(size=(experts, ff, width)) * 0.2), as_bf16(rng.normal(size=(experts, width, ff)) * 0.2)
    ids = np.stack([rng.permutation(experts)[:top] for _ in range(n)])
    weights = rng.uniform(0.05, 0.6, size=(n, top))
    got = kernels.moe_experts(device(x, dtype), device(ids, torch.int32), device(weights), device(up, dtype), device(down, dtype), False,
                              grouped=grouped, gated=False, activation="gelu_erf").cpu().numpy()
    want = np.zeros((top, n, width))
    for token in range(n):
        for choice in range(top):
            e = ids[token, choice]
            inner = plain.gelu_erf(t64(up[e]) @ t64(x[token]))
            if dtype == torch.bfloat16:
                inner = t64(as_bf16(inner.numpy()))
            want[choice, token] = weights[token, choice] * (t64(down[e]) @ inner).numpy()
    assert np.abs(got - want).max() < (3e-5 if dtype == torch.float32 else 2e-3) * max(1.0, np.abs(want).max())


# ---- the engine ---------------------------------------------------------------------------------------------------
def single_layer_folder(tmp_path, layer_of, which, with_mlp, choice=True):
    """A model of one layer: the mixer ``layer_of`` of configuration ``which``, with its own feed-forward or none."""
    import dataclasses
    from microllm_rocm_amd.config.kalevik import KalevikLayerConfig
    from microllm_rocm_amd.weights import write_model_folder
    source = CONFIGS[which] if choice else without_choice(CONFIGS[which])
    layer = source.layers[layer_of]
    if not with_mlp:
        layer = KalevikLayerConfig(layer.type, layer.mixer, None)
    config = dataclasses.replace(source, layers=(layer,), loop=None)
    folder = os.path.join(str(tmp_path), f"one_{which}_{layer_of}_{int(choice)}")
    write_model_folder(folder, config, 50 + layer_of, dtype=torch.bfloat16, stds=STDS)
    return folder


@pytest.mark.parametrize("which,layer_of,with_mlp", [("A", 0, False), ("A", 0, True), ("A", 1, False), ("A", 2, False), ("A", 3, True),
                                                     ("B", 0, False), ("B", 1, True), ("B", 2, False), ("C", 0, True), ("C", 1, False),
                                                     ("C", 2, True)])
def test_every_mixer_as_a_model_of_one_layer(tmp_path, which, layer_of, with_mlp):
    tokens = tokens_for(layer_of, 90, CONFIGS[which].vocab)
    for dtype in ("float32", "bfloat16"):
        folder = single_layer_folder(tmp_path, layer_of, which, with_mlp, choice=dtype == "float32")
        config, weights = plain.read_config(folder), plain.read_tensors(folder)
        for name, steps in (("whole", whole({"r": tokens})), ("decode", prefill_then_decode("r", tokens, tail=40)),
                            ("portions", portions("r", tokens, [2, 5, 1, 17]))):
            run_trace(folder, dtype, steps, tmp_path / f"{dtype}_{name}", max_tokens=128)
            check_against_plain(steps, tmp_path / f"{dtype}_{name}", {"r": tokens}, config, weights, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_whole_decode_and_portions(tmp_path_factory, tmp_path, which, dtype):
    folder, config, weights = model_for(tmp_path_factory, which, dtype)
    requests = {"long": tokens_for(1, 150, config["vocab"]), "short": tokens_for(2, 37, config["vocab"]), "one": tokens_for(3, 1, config["vocab"])}
    run_trace(folder, dtype, whole(requests), tmp_path / "whole", max_tokens=256)
    check_against_plain(whole(requests), tmp_path / "whole", requests, config, weights, dtype)
    for rid, tail in (("long", 70), ("short", 34)):      # the decoded tokens cross pages' and chunks' edges
        steps = prefill_then_decode(rid, requests[rid], tail=tail)
        run_trace(folder, dtype, steps, tmp_path / f"decode_{rid}", max_tokens=round_up(len(requests[rid]), 64))
        check_against_plain(steps, tmp_path / f"decode_{rid}", {rid: requests[rid]}, config, weights, dtype)
    for sizes in ([2], [3, 16, 1, 2, 31], [64, 2, 17]):
        steps = portions("long", requests["long"], sizes)
        run_trace(folder, dtype, steps, tmp_path / f"portions_{sizes[0]}", max_tokens=192)
        check_against_plain(steps, tmp_path / f"portions_{sizes[0]}", {"long": requests["long"]}, config, weights, dtype)
    steps = portions("short", requests["short"], [1])       # from its first token on, one token a step
    run_trace(folder, dtype, steps, tmp_path / "one_by_one", max_tokens=64)
    check_against_plain(steps, tmp_path / "one_by_one", {"short": requests["short"]}, config, weights, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_mixed_batches_on_reused_pages_and_slots(tmp_path_factory, tmp_path, which, dtype):
    folder, config, weights = model_for(tmp_path_factory, which, dtype)
    lengths = [90, 41, 130, 2, 67, 25, 110, 58]
    requests = {f"r{index}": tokens_for(10 + index, length, config["vocab"]) for index, length in enumerate(lengths)}
    steps, peak = mixed(requests, seed=4, max_live=3, decode_tail=12, max_portion=23)
    engine = run_trace(folder, dtype, steps, tmp_path / "mixed", max_tokens=peak, max_requests=3)
    assert all(group.pool.total_taken > group.pool.num_pages for group in engine.cache.groups)      # pages were used again
    assert engine.cache.slots.total_taken > 3                                                        # and so were slots
    check_against_plain(steps, tmp_path / "mixed", requests, config, weights, dtype)


def test_a_row_does_not_depend_on_the_batch(tmp_path_factory):
    """Float32: a request's logits are the same bits alone and beside others, whole and in portions."""
    from microllm_rocm_amd.engine import Engine, StepEntry
    folder, config, _ = model_for(tmp_path_factory, "A")
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_requests=4)
    a, b, c = (tokens_for(seed, length, config["vocab"]) for seed, length in ((1, 45), (2, 20), (3, 33)))
    engine.open("alone")
    alone = engine.step([StepEntry("alone", a, list(range(len(a))))]).clone()
    engine.close("alone")
    for name in "abc":
        engine.open(name)
    first = engine.step([StepEntry("b", b[:7], []), StepEntry("a", a[:30], list(range(30))), StepEntry("c", c[:2], [])])
    second = engine.step([StepEntry("a", a[30:44], list(range(14))), StepEntry("c", c[2:], []), StepEntry("b", b[7:8], [])])
    third = engine.step([StepEntry("b", b[8:9], [0]), StepEntry("a", a[44:], [0])])
    together = torch.cat([first, second, third[1:]])
    assert torch.equal(alone, together)


@pytest.mark.parametrize("which", ["A", "B"])
def test_long_decoding_through_graphs(tmp_path_factory, which):
    """A short prompt, then 140 tokens one by one (steps replayed from captured graphs, state carried in slots, cached
    rows crossing many pages and chunks), two requests at once with unequal lengths."""
    from microllm_rocm_amd.engine import Engine, StepEntry
    folder, config, weights = model_for(tmp_path_factory, which)
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_requests=2)
    assert engine.use_graphs
    sequences = {"x": tokens_for(7, 150, config["vocab"]), "y": tokens_for(8, 160, config["vocab"])}
    starts = {"x": 10, "y": 3}
    rows = {name: [] for name in sequences}
    for name in sequences:
        engine.open(name)
    logits = engine.step([StepEntry(name, sequences[name][:starts[name]], [starts[name] - 1]) for name in sequences])
    for index, name in enumerate(sequences):
        rows[name].append(logits[index].cpu().numpy())
    for offset in range(140):
        entries = [StepEntry(name, [sequences[name][starts[name] + offset]], [0]) for name in sequences]
        logits = engine.step(entries)
        for index, name in enumerate(sequences):
            rows[name].append(logits[index].cpu().numpy())
    assert engine.graph_replays >= 139
    for name, tokens in sequences.items():
        want = plain_logits(config, weights, tokens[:starts[name] + 140])[starts[name] - 1:]
        sensitivity = plain_run(config, weights, tokens[:starts[name] + 140])[3][starts[name] - 1:]
        assert (row_errors(np.stack(rows[name]), want) / sensitivity).max() < F32_BOUND


@pytest.mark.parametrize("which", ["A", "C"])
def test_greedy_generation_through_the_scheduler(tmp_path_factory, which):
    from microllm_rocm_amd import Engine, GenerationConfig, generate, generate_serial
    folder, config, weights = model_for(tmp_path_factory, which)
    prompts = [tokens_for(20 + index, length, config["vocab"]) for index, length in enumerate((5, 31, 12))]
    expected = [prompt + plain.generate_greedy(config, weights, prompt, 10) for prompt in prompts]
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=512, max_requests=4)
    got = generate(engine, prompts, GenerationConfig(max_new_tokens=10, temperature=0.0), prefill_chunk=7, max_batched_tokens=16)
    assert got == expected
    assert generate_serial(engine, prompts[0], GenerationConfig(max_new_tokens=10, temperature=0.0)) == expected[0]
    bf16 = Engine.from_folder(folder, dtype="bfloat16", max_tokens=512, max_requests=4)
    close = generate(bf16, prompts, GenerationConfig(max_new_tokens=10, temperature=0.0), prefill_chunk=7)
    assert [len(tokens) for tokens in close] == [len(tokens) for tokens in expected]
    assert all(tokens[:len(prompt)] == prompt for tokens, prompt in zip(close, prompts))


@pytest.mark.parametrize("which", ["A", "B", "C"])
def test_residual_stream_after_every_layer_run(tmp_path_factory, tmp_path, which):
    """A looped layer counts each time it runs; the embedding's output that a later pass begins with is not yet in the
    stream the pass before leaves."""
    folder, config, weights = model_for(tmp_path_factory, which)
    tokens = tokens_for(5, 19, config["vocab"])
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": tokens, "want": list(range(19))}], "end": ["q"]}]
    from microllm_rocm_amd.engine import Engine
    from microllm_rocm_amd.engine.replay import replay
    engine = Engine.from_folder(folder, dtype="float32", max_tokens=64, max_requests=1)
    replay(engine, io.StringIO(to_lines(steps)), str(tmp_path), io.StringIO(), dump_layers=True)
    streams = plain_run(config, weights, tokens)[1]
    runs = len(plain.run_order(config))
    assert streams.shape[0] == runs
    got = np.fromfile(os.path.join(str(tmp_path), "0.layers.f32"), dtype="<f4").reshape(runs, 19, config["width"])
    for run in range(runs):
        assert np.abs(got[run] - streams[run]).max() < 1e-4 * np.abs(streams[run]).max(), run


def test_plain_pages_in_bfloat16(tmp_path_factory):
    """A bfloat16 engine whose attention layers are told not to take the MFMA kernels runs the same model on plain
    pages; it stays within the format's cost of the plain run, decoding across chunks."""
    import dataclasses
    from microllm_rocm_amd.config.registry import load_config
    from microllm_rocm_amd.engine import Engine, StepEntry
    from microllm_rocm_amd.parts import Model, PartSpec, Runtime
    from microllm_rocm_amd.weights import load_folder
    folder, config, weights = model_for(tmp_path_factory, "C", "bfloat16")
    architecture, typed = load_config(folder)
    spec = architecture.build_spec(typed)

    def unmatrixed(mixer):
        if mixer.kind == "parallel":
            return PartSpec(mixer.kind, {"members": tuple((unmatrixed(member), scale) for member, scale in mixer.params["members"])}, mixer.names)
        if mixer.kind in ("latent_attention", "bucket_bias_attention"):
            return PartSpec(mixer.kind, {**mixer.params, "mfma": False}, mixer.names)
        return mixer

    spec = dataclasses.replace(spec, layers=tuple(dataclasses.replace(layer, mixer=unmatrixed(layer.mixer)) for layer in spec.layers))
    probe = Model(spec, Runtime(torch.bfloat16, torch.device("cpu")))
    assert not any(getattr(part, "tiled", False) for part in probe.parts())
    tiled = Model(architecture.build_spec(typed), Runtime(torch.bfloat16, torch.device("cpu")))
    assert sum(bool(getattr(part, "tiled", False)) for part in tiled.parts()) == 2      # as built, both take the MFMA kernels
    tensors = load_folder(folder, probe.tensors(), torch.bfloat16, torch.device("cuda:0"))
    engine = Engine(spec, tensors, dtype="bfloat16", max_tokens=256, max_requests=2, tensors_placed=True)
    tokens = tokens_for(9, 120, config["vocab"])
    engine.open("p")
    first = engine.step([StepEntry("p", tokens[:40], list(range(40)))]).cpu().numpy()
    rest = [engine.step([StepEntry("p", [token], [0])]).cpu().numpy() for token in tokens[40:]]
    got = np.concatenate([first] + rest)
    _, _, margin, sensitivity = plain_run(config, weights, tokens)
    errors = row_errors(got, plain_logits(config, weights, tokens)) / sensitivity
    assert within_bound(np.where(margin >= ROUTER_MARGIN, errors, 0.0), "bfloat16")


def test_command_line_and_trace_runner_as_programs(tmp_path_factory, tmp_path, capsys):
    import json
    import subprocess
    import sys
    from microllm_rocm_amd.cli import hf_infer
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, config, weights = model_for(tmp_path_factory, "A")
    prompt = tokens_for(31, 13, config["vocab"])
    expected = plain.generate_greedy(config, weights, prompt, 6)
    base = ["--model", folder, "--tokens", ",".join(map(str, prompt)), "--new-tokens", "6", "--dtype", "float32"]

    def run(*more):
        capsys.readouterr()
        assert hf_infer.main(base + list(more)) == 0
        return json.loads(capsys.readouterr().out.strip().splitlines()[-1])

    report = run()
    assert report["architecture"] == "Kalevik" and report["generated_tokens"] == expected
    for more in (["--use-cache", "false"], ["--cache-prefill-mode", "token"], ["--batch", "2", "--batch-argmax-mode", "host"]):
        assert run(*more)["generated_tokens"] == expected, more
    sampled = [run("--temperature", "0.9", "--sample-top-k", "5", "--seed", "7")["generated_tokens"] for _ in range(2)]
    assert sampled[0] == sampled[1] and len(sampled[0]) == 6
    steps = portions("p", prompt + expected, [5, 2, 1])
    result = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out",
                             str(tmp_path / "trace"), "--max-tokens", "64"], input=to_lines(steps), capture_output=True, text=True, timeout=300)
    assert result.returncode == 0, result.stderr
    assert [line for line in result.stdout.splitlines() if line.startswith("done")] == [f"done {step['step']}" for step in steps]
    check_against_plain(steps, tmp_path / "trace", {"p": prompt + expected}, config, weights, "float32")
