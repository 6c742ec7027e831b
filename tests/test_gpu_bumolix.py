"""Bumolix models through the engine against the plain implementation (tests/plain/bumolix_plain.py):
every way of cutting the work, batches, pages and state slots used again, keys far back in a
chunk and on either side of a chunk's edge, the sink, the first tokens, recurrences that
remember, long decoding, and greedy generation through ``Engine.generate``.  Small configurations
of the tests' own, random weights; where random weights would hide a fault the scores are made
sharp or one mixer is switched off by its scale."""
import json
import os
import subprocess

import numpy as np
import pytest

from bumolix_util import (CFG_A, CFG_B, CFG_C, config, dense, left, parallel_layer, random_weights, right, scan_layer,
                          write_model)
from conftest import ROOT
from gpu_util import chunked_steps, make_runner, mixed_steps, run_steps, tail_decode_steps, whole_steps
from plain import bumolix_plain as P

pytestmark = pytest.mark.gpu

CONFIGS = {"A": (CFG_A, 21), "B": (CFG_B, 22), "C": (CFG_C, 23)}
LENGTHS = {"A": [70, 1, 45, 2, 90, 33, 58], "B": [40, 75, 3, 52, 21], "C": [30, 64, 17, 49, 5]}
PAGE = {"A": 4, "B": 8, "C": 16}      # A's chunks of 12 and 7 and C's of 5 end inside pages


def tokens_of(vocab, n, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, (cfg, seed) in CONFIGS.items():
        w = random_weights(cfg, seed)
        streams = {f"r{i}": tokens_of(cfg["vocab"], n, 50 + i) for i, n in enumerate(LENGTHS[name])}
        refs = {r: P.forward(cfg, w, t, np.float64) for r, t in streams.items()}
        for dtype in ("float32", "bfloat16"):
            folder = write_model(str(tmp_path_factory.mktemp(f"bumolix{name}_{dtype}")), cfg, w, dtype)
            out[(name, dtype)] = (folder, streams, refs)
    return out


def assert_close(got, want, dtype, what=""):
    """Against the float64 values, relative to the largest logit.  float32 differs by the order of
    its sums alone.  bfloat16 rounds every product's inputs, and narrow random models with
    recurrences amplify that: nine rows in ten within 5 %, every row within 20 %; a wrong key,
    a lost state or a sink left out moves most rows by the logits' own size."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, f"{what}: shape {got.shape} vs {want.shape}"
    err = np.abs(got - want).reshape(len(want), -1).max(axis=1) / max(1.0, np.abs(want).max())
    ok = err.max() <= 3e-5 if dtype == "float32" else (err.max() <= 0.20 and np.quantile(err, 0.9) <= 0.05)
    if not ok:
        raise AssertionError(f"{what}: largest relative error {err.max():.3e} at row {int(np.argmax(err))}, "
                             f"nine in ten below {np.quantile(err, 0.9):.3e}")


def check(rows, refs, dtype, what):
    assert set(rows) == set(refs)
    for r in refs:
        assert_close(rows[r], refs[r], dtype, f"{what} {r}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_every_split_matches_the_plain_implementation(models, name, dtype):
    folder, streams, refs = models[(name, dtype)]
    runner = make_runner(folder, dtype, page_size=PAGE[name], cache_tokens=128, max_seqs=2, max_batch_tokens=128,
                         max_model_len=128)
    whole = run_steps(runner, streams, whole_steps(streams))
    check(whole, refs, dtype, "whole")
    tail = run_steps(runner, streams, tail_decode_steps(streams, tail=40))
    check(tail, refs, dtype, "last 40 one by one")
    one = run_steps(runner, streams, tail_decode_steps(streams, tail=1000))
    check(one, refs, dtype, "token by token")
    chunk = run_steps(runner, streams, chunked_steps(streams))
    check(chunk, refs, dtype, "portions")
    pairs = run_steps(runner, streams, chunked_steps(streams, sizes=(2,)))
    check(pairs, refs, dtype, "portions of two")
    if dtype == "float32":
        # every sum runs in an order fixed by positions and channels alone: the cuts change nothing
        for r in streams:
            for other in (tail, one, chunk, pairs):
                assert np.array_equal(whole[r], other[r]), r
    assert all(p.free_pages == p.num_pages for p in runner.manager.pools)
    assert runner.manager.slots.free_slots == 2


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C"])
def test_mixed_batches_with_pages_and_slots_used_again(models, name, dtype):
    folder, streams, refs = models[(name, dtype)]
    page = PAGE[name]
    pages_of = lambda n: -(-n // page)
    room = sum(sorted((pages_of(len(t)) for t in streams.values()), reverse=True)[:3])
    runner = make_runner(folder, dtype, page_size=page, num_pages=room, max_seqs=3, max_batch_tokens=128,
                         max_model_len=128)
    alone = run_steps(runner, streams, whole_steps(streams))
    for seed in (0, 1):
        steps = mixed_steps(streams, seed=seed, max_live=3, room=room, page=page, decode_tail=9)
        assert any(any(n > 1 for _, n in e) and any(n == 1 for _, n in e) for e, _ in steps)
        slots_seen = {}

        def observe(_):
            for r in runner.manager.live():
                slots_seen.setdefault(runner.manager.slot(r), set()).add(r)

        rows = run_steps(runner, streams, steps, observe)
        check(rows, refs, dtype, f"mixed seed {seed}")
        assert any(len(v) >= 2 for v in slots_seen.values()), "no state slot was used again"
        if dtype == "float32":
            for r in streams:
                assert np.array_equal(rows[r], alone[r]), f"{r} differs from its run alone"
    assert all(p.free_pages == p.num_pages for p in runner.manager.pools)


def test_a_chunked_attention_gives_pages_back_while_a_request_runs(models):
    """A pool too small for a request's whole length serves it all the same: pages before the
    current chunk come back as the request moves on, and are handed out again."""
    cfg = config([parallel_layer(left(2, 1, 16, 16, chunk=16, rot_dims=8), right(2, 8, 8, 4.0, 4), mlp=dense(24))], vocab=40, width=32)
    w = random_weights(cfg, 5)
    toks = tokens_of(40, 120, 1)
    ref = P.forward(cfg, w, toks, np.float64)
    import tempfile
    with tempfile.TemporaryDirectory() as d:
        folder = write_model(d, cfg, w, "float32")
        # three chunks' worth of pages for a request of 120 tokens
        runner = make_runner(folder, "float32", page_size=4, num_pages=12, max_seqs=1, max_batch_tokens=32, max_model_len=128)
        rows = run_steps(runner, {"r": toks}, chunked_steps({"r": toks}, sizes=(9, 1, 1, 30, 2, 7)))
        assert_close(rows["r"], ref, "float32", "a small pool")
        assert all(p.free_pages == p.num_pages for p in runner.manager.pools)


# ---------------------------------------------------------------- keys far back, chunk edges, the sink
def attention_alone(chunk, dtype, tmp_path, right_scale=0.0, **kw):
    """One layer whose right mixer is switched off by its scale and that has no feed-forward: the
    logits at a position follow from the tokens of its chunk alone.  Queries and keys are unit
    vectors times sqrt(dim) whatever the projections' size, so the config's scale sets how sharp
    the softmax is: 2 on heads of 16 gives scores of up to 32, close to a choice of one key."""
    l = left(kw.pop("heads", 2), kw.pop("kv_heads", 1), kw.pop("dim", 16), kw.pop("vdim", 24), chunk=chunk,
             rot_dims=kw.pop("rot_dims", 8), base=30.0, factor=2.0, scale=kw.pop("scale", 2.0))
    cfg = config([parallel_layer(l, right(1, 8, 8, 2.0, 2), 3.0, right_scale, None)], vocab=50, width=32, mult=1.0)
    w = random_weights(cfg, 11)
    return cfg, w, write_model(str(tmp_path / f"alone_{chunk}_{dtype}"), cfg, w, dtype)


# head shapes: values of another size than keys run on the plain attention kernel in either type,
# equal sizes of 16, 32, ... on the matrix-core kernel in bfloat16 (the far key of this draw shows with heads of 16)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim,vdim", [(16, 24), (16, 16)])
def test_a_key_hundreds_of_tokens_back_in_its_chunk(tmp_path, dim, vdim, dtype):
    cfg, w, folder = attention_alone(400, dtype, tmp_path, dim=dim, vdim=vdim)
    n = 390
    base = tokens_of(cfg["vocab"], n, 21)
    ref = P.forward(cfg, w, base, np.float64)
    # the early token whose change moves the last logits most is the far key
    moved = {}
    for j in range(5, 60):
        t = list(base)
        t[j] = (t[j] + 7) % cfg["vocab"]
        moved[j] = np.abs(P.forward(cfg, w, t, np.float64)[-1] - ref[-1]).max()
    far = max(moved, key=moved.get)
    assert moved[far] > 0.05 * np.abs(ref[-1]).max(), "no far key matters in this draw"
    other = list(base)
    other[far] = (other[far] + 7) % cfg["vocab"]
    ref_other = P.forward(cfg, w, other, np.float64)
    runner = make_runner(folder, dtype, page_size=16, cache_tokens=2 * 400, max_seqs=2, max_batch_tokens=512, max_model_len=400)
    streams = {"base": base, "other": other}
    for how, steps in (("prompt", whole_steps(streams)), ("decoded", tail_decode_steps(streams, tail=20)),
                       ("portions", chunked_steps(streams, sizes=(64, 3, 31, 2)))):
        rows = run_steps(runner, streams, steps)
        assert_close(rows["base"], ref, dtype, f"{how} base")
        assert_close(rows["other"], ref_other, dtype, f"{how} other")
        assert np.abs(rows["other"][-1] - rows["base"][-1]).max() > 0.02 * np.abs(ref[-1]).max(), how


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("vdim", [24, 16])
@pytest.mark.parametrize("chunk,page", [(12, 8), (7, 4), (40, 16), (16, 16), (33, 4)])
def test_keys_just_inside_and_just_outside_a_chunks_edge(tmp_path, chunk, page, vdim, dtype):
    """With the attention alone, a change of the last token before a chunk must leave every logit
    of the chunk as it was, to the bit, and a change of the chunk's first token must move them
    as the plain implementation says; in prompts, in portions that end and begin at and around
    the edge, and token by token."""
    cfg, w, folder = attention_alone(chunk, dtype, tmp_path, vdim=vdim)
    n = 3 * chunk + chunk // 2
    base = tokens_of(cfg["vocab"], n, 3)
    edge = 2 * chunk
    outside, inside = list(base), list(base)
    outside[edge - 1] = (outside[edge - 1] + 9) % cfg["vocab"]
    inside[edge] = (inside[edge] + 9) % cfg["vocab"]
    streams = {"base": base, "outside": outside, "inside": inside}
    refs = {r: P.forward(cfg, w, t, np.float64) for r, t in streams.items()}
    assert np.abs(refs["outside"][edge:] - refs["base"][edge:]).max() < 1e-9
    seen = np.abs(refs["inside"][edge + 1:3 * chunk] - refs["base"][edge + 1:3 * chunk]).max(axis=1)
    assert (seen > 0.02 * np.abs(refs["base"]).max()).any(), "the chunk's first key matters to none in this draw"
    runner = make_runner(folder, dtype, page_size=page, cache_tokens=3 * 256, max_seqs=3, max_batch_tokens=256, max_model_len=256)
    ways = (("prompt", whole_steps(streams)),
            ("decoded", tail_decode_steps(streams, tail=n - edge + 3)),
            ("token by token", tail_decode_steps(streams, tail=1000)),
            ("portions", chunked_steps(streams, sizes=(edge - 1, 2, chunk - 1, 3, 2))),
            ("portions to the edge", chunked_steps(streams, sizes=(edge, 1, chunk - 1, 2))))
    for how, steps in ways:
        rows = run_steps(runner, streams, steps)
        check(rows, refs, dtype, how)
        assert np.array_equal(rows["outside"][edge:], rows["base"][edge:]), f"{how}: a key before the chunk was read"
        assert np.abs(rows["inside"][edge:3 * chunk] - rows["base"][edge:3 * chunk]).max() > 0.01 * np.abs(refs["base"]).max(), how


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("vdim", [8, 16])
def test_the_sink_takes_its_share_of_the_weights(tmp_path, vdim, dtype):
    """Scores of either sign and several units: a query whose keys all score low gives most of its
    weight to the sink, one with a high score nearly nothing.  Left out of the denominator, or
    given a value, the sink would move every such row."""
    cfg, w, folder = attention_alone(9, dtype, tmp_path, scale=0.5, heads=3, kv_heads=3, vdim=vdim)
    toks = tokens_of(cfg["vocab"], 50, 5)
    x = P.rms_norm(w["embed"][toks].astype(np.float64), w["l0.norm1"], cfg["norm"]["eps"], np.float64)
    m = cfg["layers"][0]["mixer"]["left"]
    with_sink = P.left_mixer(x, np.arange(50), w, "l0.mix.left.", m, cfg["norm"]["eps"], np.float64)
    # the same mixer with an ordinary softmax, through the plain functions
    def no_sink(q, k, v, scale, seen, dt, sink=True):
        return real(q, k, v, scale, seen, dt, sink=False)
    real, P.sink_softmax_attention = P.sink_softmax_attention, no_sink
    try:
        without = P.left_mixer(x, np.arange(50), w, "l0.mix.left.", m, cfg["norm"]["eps"], np.float64)
    finally:
        P.sink_softmax_attention = real
    share = np.linalg.norm(with_sink, axis=1) / np.linalg.norm(without, axis=1)
    assert (share < 0.8).sum() >= 5 and (share > 0.9).sum() >= 5, "the sink neither wins nor loses in this draw"
    ref = P.forward(cfg, w, toks, np.float64)
    runner = make_runner(folder, dtype, page_size=8, cache_tokens=128, max_seqs=1, max_batch_tokens=64, max_model_len=64)
    for steps in (whole_steps({"r": toks}), tail_decode_steps({"r": toks}, tail=30), chunked_steps({"r": toks})):
        assert_close(run_steps(runner, {"r": toks}, steps)["r"], ref, dtype, "sink")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("kind", ["decayed", "scan"])
def test_the_recurrence_remembers_the_first_tokens(tmp_path, kind, dtype):
    """Decays close to one: what the recurrence took in at the start still shows two hundred
    tokens later, through a state carried over portions and single tokens, although the
    attention beside it sees its own chunk only."""
    if kind == "decayed":
        cfg = config([parallel_layer(left(2, 1, 8, 8, chunk=10, rot_dims=4), right(2, 16, 12, 8.0, 4), 0.5, 1.5, None)],
                     vocab=50, width=32, mult=1.0)
        w = random_weights(cfg, 42)
        w["l0.mix.right.a2.b"][:] = 6.0
    else:
        cfg = config([scan_layer(24, 8, 4, 3, None)], vocab=50, width=32, mult=1.0)
        w = random_weights(cfg, 42)
        w["l0.mix.A_log"][:] = -5.0
    n = 200
    base = tokens_of(cfg["vocab"], n, 9)
    other = [(t + 11) % cfg["vocab"] for t in base[:6]] + base[6:]
    ref, ref_other = P.forward(cfg, w, base, np.float64), P.forward(cfg, w, other, np.float64)
    assert np.abs(ref_other[-1] - ref[-1]).max() > 0.01 * np.abs(ref[-1]).max(), "the start is forgotten in this draw"
    folder = write_model(str(tmp_path / f"memory_{kind}_{dtype}"), cfg, w, dtype)
    runner = make_runner(folder, dtype, page_size=16, cache_tokens=1024, max_seqs=2, max_batch_tokens=512, max_model_len=512)
    streams = {"base": base, "other": other}
    for how, steps in (("prompt", whole_steps(streams)), ("decoded", tail_decode_steps(streams, tail=180)),
                       ("portions", chunked_steps(streams, sizes=(17, 2, 40, 1, 16)))):
        rows = run_steps(runner, streams, steps)
        assert_close(rows["base"], ref, dtype, f"{how} base")
        assert_close(rows["other"], ref_other, dtype, f"{how} other")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("segment", [16, 64])
def test_long_portions_walked_in_segments(tmp_path, monkeypatch, segment, dtype):
    """Few long portions: the recurrences walk segments of a portion side by side and join them.
    Portions that end inside a segment, on its edge and one past it, beside a short one; later
    portions start from the state the earlier ones left; decays near one and far from it."""
    from zse_amd.parts.gla import GatedLinearAttention
    from zse_amd.parts.scan import SelectiveScan
    monkeypatch.setattr(GatedLinearAttention, "SEGMENT", segment)
    monkeypatch.setattr(SelectiveScan, "SEGMENT", segment)
    cfg = config([parallel_layer(left(2, 1, 8, 8, chunk=24, rot_dims=4), right(3, 12, 40, 2.0, 4), 0.6, 1.4, dense(24)),
                  scan_layer(72, 5, 3, 3, None),
                  parallel_layer(left(1, 1, 16, 16, chunk=9, rot_dims=8), right(1, 40, 24, 9.0, 2), 1.0, 1.0, None)],
                 vocab=70, width=40, mult=0.6)
    w = random_weights(cfg, 31)
    w["l0.mix.right.a2.b"][:] = np.linspace(-4.0, 8.0, 36)
    w["l1.mix.A_log"][:] = np.linspace(-5.0, 1.5, 72 * 5).reshape(72, 5)
    lengths = {"a": 4 * segment + 7, "b": 2 * segment, "c": 2 * segment + 1, "d": 5, "e": 3 * segment - 1}
    streams = {r: tokens_of(cfg["vocab"], n, 60 + i) for i, (r, n) in enumerate(lengths.items())}
    refs = {r: P.forward(cfg, w, t, np.float64) for r, t in streams.items()}
    folder = write_model(str(tmp_path / f"segments_{segment}_{dtype}"), cfg, w, dtype)
    runner = make_runner(folder, dtype, page_size=8, cache_tokens=1024, max_seqs=3, max_batch_tokens=1024, max_model_len=512)
    check(run_steps(runner, streams, whole_steps(streams)), refs, dtype, "whole")
    # a, b and d in one step, then c and e with what is left of nothing: three requests of unequal length a step
    together = [([("a", lengths["a"]), ("b", lengths["b"]), ("d", lengths["d"])], ["a", "b", "d"]),
                ([("c", lengths["c"]), ("e", lengths["e"])], ["c", "e"])]
    check(run_steps(runner, streams, together), refs, dtype, "unequal requests together")
    sizes = (2 * segment + 3, 2, 2 * segment, 1, 3 * segment)
    check(run_steps(runner, streams, chunked_steps(streams, sizes=sizes)), refs, dtype, "long portions one after the other")
    assert runner.manager.slots.free_slots == 3


def test_decays_far_from_one_and_steps_of_every_size(tmp_path):
    """tau = 1 with strongly negative arguments forgets within a token or two, large steps of the
    scan saturate exp(step A): the 32-bit arithmetic of decays, logarithms and softplus holds at
    both ends."""
    cfg = config([parallel_layer(left(chunk=6), right(2, 8, 8, 1.0, 3), 1.0, 1.0, dense(16)), scan_layer(16, 4, 3, 2, None)],
                 vocab=40, width=32, mult=0.5)
    w = random_weights(cfg, 8)
    w["l0.mix.right.a2.b"][:] = np.linspace(-12.0, 12.0, 16)
    w["l1.mix.dt.b"][:] = np.linspace(-9.0, 6.0, 16)
    w["l1.mix.A_log"][:] = np.linspace(-4.0, 2.5, 64).reshape(16, 4)
    toks = tokens_of(40, 60, 4)
    ref = P.forward(cfg, w, toks, np.float64)
    folder = write_model(str(tmp_path / "ends"), cfg, w, "float32")
    runner = make_runner(folder, "float32", page_size=8, cache_tokens=64, max_seqs=1, max_batch_tokens=64, max_model_len=64)
    for steps in (whole_steps({"r": toks}), tail_decode_steps({"r": toks}, tail=50), chunked_steps({"r": toks}, sizes=(19, 2, 3))):
        assert_close(run_steps(runner, {"r": toks}, steps)["r"], ref, "float32", "both ends")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_through_every_kind_of_state(models, dtype):
    cfg, seed = CONFIGS["A"]
    folder = models[("A", dtype)][0]
    w = random_weights(cfg, seed)
    toks = tokens_of(cfg["vocab"], 240, 77)
    ref = P.forward(cfg, w, toks, np.float64)
    runner = make_runner(folder, dtype, page_size=4, cache_tokens=256, max_seqs=1, max_batch_tokens=64, max_model_len=256)
    rows = run_steps(runner, {"r": toks}, tail_decode_steps({"r": toks}, tail=230))
    assert_close(rows["r"], ref, dtype, "230 tokens one by one")


def test_the_first_tokens_of_a_sequence(models):
    """Positions 0 to 3: the convolution reads rows before the sequence (zeros), the recurrences
    start from zero states, the sink outweighs the one or two keys there are."""
    for name in ("A", "B", "C"):
        cfg, seed = CONFIGS[name]
        folder = models[(name, "float32")][0]
        w = random_weights(cfg, seed)
        runner = make_runner(folder, "float32", page_size=4, cache_tokens=64, max_seqs=2, max_batch_tokens=64, max_model_len=64)
        for n in (1, 2, 3, 4):
            toks = tokens_of(cfg["vocab"], n, 200 + n)
            ref = P.forward(cfg, w, toks, np.float64)
            for steps in (whole_steps({"r": toks}), tail_decode_steps({"r": toks}, tail=10)):
                rows = run_steps(runner, {"r": toks}, steps)
                assert_close(rows["r"], ref, "float32", f"{name}: {n} tokens")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_slot_taken_over_starts_from_zero(models, dtype):
    """One slot, requests one after the other: none must see what the one before left in the
    states or in the convolution's rows."""
    folder, streams, refs = models[("A", dtype)]
    runner = make_runner(folder, dtype, page_size=4, cache_tokens=128, max_seqs=1, max_batch_tokens=128, max_model_len=128)
    for r in ("r0", "r4", "r2", "r0"):
        rows = run_steps(runner, {r: streams[r]}, chunked_steps({r: streams[r]}, sizes=(9, 1, 4)))
        assert_close(rows[r], refs[r], dtype, r)


def test_the_states_of_a_layer_lie_one_behind_the_other(models):
    """A parallel layer's right mixer keeps its state in the request's slot beside the pages of
    the left one; a scan keeps S and the convolution's rows: no two layers share words."""
    folder = models[("A", "float32")][0]
    runner = make_runner(folder, "float32", page_size=4, cache_tokens=64, max_seqs=2, max_batch_tokens=64, max_model_len=64)
    spans = sorted((c.state_offset, c.state_offset + c.state_bytes) for c in runner.caches if c.state_bytes)
    assert len(spans) == 4
    assert all(a[1] <= b[0] for a, b in zip(spans, spans[1:]))


# ---------------------------------------------------------------- the engine's own entry point
def plain_greedy(cfg, w, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(P.forward(cfg, w, toks, np.float64)[-1])))
    return toks[len(prompt):]


def test_greedy_generation_through_the_engine(models):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling.sampler import SamplingParams
    cfg, seed = CONFIGS["A"]
    folder = models[("A", "float32")][0]
    w = random_weights(cfg, seed)
    prompts = [tokens_of(cfg["vocab"], n, 300 + n) for n in (5, 23, 1, 40, 12, 31)]
    want = [plain_greedy(cfg, w, p, 12) for p in prompts]
    # four places for six requests, portions of 16: prompts are cut, requests wait for a slot
    with Engine(folder, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=32, max_batch_seqs=4,
                prefill_chunk_size=16, max_seq_len=128) as eng:
        got = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0))
        assert got == want
        again = eng.generate(prompts[:2], SamplingParams(max_tokens=12, temperature=0.0))
        assert again == want[:2]
    with Engine(folder, dtype="float32", block_size=4, num_blocks=64, max_batch_tokens=32, max_batch_seqs=4,
                prefill_chunk_size=16, max_seq_len=128, use_graphs=False) as eng:
        assert eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0)) == want


def test_generation_in_bfloat16_through_graphs_does_not_depend_on_the_company(models):
    from zse_amd.engine.engine import Engine
    from zse_amd.sampling.sampler import SamplingParams
    cfg, _ = CONFIGS["B"]
    folder = models[("B", "bfloat16")][0]
    prompts = [tokens_of(cfg["vocab"], n, 400 + n) for n in (9, 30, 17)]
    sp = SamplingParams(max_tokens=10, temperature=0.0)
    with Engine(folder, dtype="bfloat16", block_size=8, num_blocks=64, max_batch_tokens=64, max_batch_seqs=4,
                prefill_chunk_size=64, max_seq_len=128) as eng:
        together = eng.generate(prompts, sp)
        alone = [eng.generate([p], sp)[0] for p in prompts]
        assert eng.runner.graph_runs > 0, "no decode step was replayed from a graph"
    assert together == alone
    with Engine(folder, dtype="bfloat16", block_size=8, num_blocks=64, max_batch_tokens=64, max_batch_seqs=4,
                prefill_chunk_size=64, max_seq_len=128, use_graphs=False) as eng:
        assert eng.generate(prompts, sp) == together


def test_the_trace_program_serves_the_design(models, tmp_path):
    cfg, seed = CONFIGS["B"]
    folder, streams, refs = models[("B", "float32")]
    out = tmp_path / "out"
    a, b = streams["r0"], streams["r1"]
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:7], "want": [0, 6]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[7:9], "want": []}, {"id": "b", "tokens": b[:40], "want": [39]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[40:41], "want": [0]}, {"id": "a", "tokens": a[9:], "want": [len(a) - 10]}],
         "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b[41:], "want": [len(b) - 42]}], "end": ["b"]},
    ]
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "128"], input="\n".join(json.dumps(s) for s in steps) + "\n",
                       capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    V = cfg["vocab"]
    read = lambda i: np.fromfile(str(out / f"{i}.f32"), dtype="<f4").reshape(-1, V)
    assert_close(read(0), refs["r0"][[0, 6]], "float32", "step 0")
    assert_close(read(1), refs["r1"][[39]], "float32", "step 1")
    assert_close(read(2), np.stack([refs["r1"][40], refs["r0"][len(a) - 1]]), "float32", "step 2")
    assert_close(read(3), refs["r1"][[len(b) - 1]], "float32", "step 3")
