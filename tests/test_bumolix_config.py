"""Bumolix on the host: registry, configuration keys, the tensor list, what a request keeps (pages
of a chunked attention, states behind them), which pages a chunk gives back, divided
frequencies, what the config leaves out, error messages, and the plain implementation's own
mechanisms against closed forms."""
import copy

import numpy as np
import pytest

import zse_amd.models  # noqa: F401
from bumolix_util import CFG_A, CFG_B, CFG_C, config, dense, left, parallel_layer, right, scan_layer, tensor_shapes
from plain import bumolix_plain as P
from zse_amd.config.base import ConfigError, resolve_architecture
from zse_amd.engine.model import Model
from zse_amd.parts.base import PagedKV, StateNeed


def model_of(cfg):
    arch = resolve_architecture(cfg)
    return Model(arch.plan(arch.config_from_dict(cfg)))


def test_the_registry_knows_the_design():
    assert resolve_architecture({"architecture": "Bumolix"}).name == "Bumolix"
    assert resolve_architecture({"model_type": "bumolix"}).name == "Bumolix"


@pytest.mark.parametrize("cfg", [CFG_A, CFG_B, CFG_C])
def test_the_model_asks_for_exactly_the_checkpoints_tensors(cfg):
    reqs = {r.name: tuple(r.shape) for r in model_of(cfg).tensor_reqs()}
    want = tensor_shapes(cfg)
    # the rank of the decays' projection is no key of the format: the model leaves it open (-1)
    # unless a config names it, and reads it off the tensors when it loads them
    for name, shape in reqs.items():
        assert name in want, name
        assert all(a == b or a == -1 for a, b in zip(shape, want[name])) and len(shape) == len(want[name]), name
    assert set(reqs) == set(want)


def test_what_a_request_keeps():
    needs = model_of(CFG_A).cache_needs()
    assert [type(n) for n in needs] == [PagedKV, StateNeed, PagedKV, StateNeed]
    # pages of the left mixer, chunked; the right mixer's S [heads, dim, vdim] as floats beside them
    assert (needs[0].num_kv_heads, needs[0].head_dim, needs[0].value_dim, needs[0].window, needs[0].chunk) == (2, 16, 24, None, 12)
    assert needs[0].state_bytes == 4 * 3 * 8 * 12
    assert (needs[2].num_kv_heads, needs[2].head_dim, needs[2].value_dim, needs[2].chunk) == (2, 8, None, 7)
    assert needs[2].state_bytes == 4 * 2 * 20 * 10
    # S [inner, state] as floats, then taps - 1 rows of the convolution's inputs
    assert needs[1].nbytes == 4 * (24 * 6 + 2 * 24)
    assert needs[3].nbytes == 4 * (40 * 17 + 3 * 40)
    c = model_of(CFG_C).cache_needs()
    assert c[1].nbytes == 4 * 9 * 1                    # one tap: nothing of the convolution is kept
    assert c[2].chunk is None and c[2].window is None  # no mask: every key stays


def test_layers_with_different_chunks_keep_their_pages_apart():
    from zse_amd.cache.manager import group_needs
    groups = group_needs(model_of(CFG_A).cache_needs())
    assert [(g.window, g.chunk, g.calls) for g in groups] == [(None, 7, [2]), (None, 12, [0])]
    mixed = config([parallel_layer(left(chunk=None)), parallel_layer(left(chunk=12)), scan_layer(), parallel_layer(left(chunk=12))])
    groups = group_needs(model_of(mixed).cache_needs())
    assert [(g.chunk, g.calls) for g in groups] == [(12, [1, 3]), (None, [0])]


@pytest.mark.parametrize("chunk,page", [(12, 4), (7, 4), (5, 16), (32, 8), (9, 3)])
def test_a_chunk_gives_back_the_pages_before_it(chunk, page):
    """After n tokens are computed, the next query sits at position n: every page whose newest key
    lies before floor(n / chunk) * chunk is free, every other page is held."""
    from zse_amd.cache.manager import CacheManager, GroupInfo
    m = CacheManager([GroupInfo(None, [0], num_pages=64, chunk=chunk)], page_size=page, max_seqs=1, max_model_len=64)
    m.add("r")
    for n in range(1, 60):
        m.reserve("r", n)
        m.commit("r", n)
        first = n // chunk * chunk
        held = [j for j, p in enumerate(m.table("r", 0)) if p >= 0]
        want = [j for j in range(-(-n // page)) if (j + 1) * page - 1 >= first]
        assert held == want, (n, held, want)
        m.check()
    m.release("r")
    assert m.pools[0].free_pages == 64


def test_divided_frequencies():
    m = model_of(CFG_A)
    rot = m.blocks[0].mixer.mixers[0].position
    assert np.allclose(rot.frequencies(), P.rotary_frequencies(8, 500.0, 4.0).astype(np.float32), rtol=1e-6)
    assert rot.magnitude() == 1.0 and not rot.interleaved
    whole = model_of(CFG_B).blocks[1].mixer.mixers[0].position
    assert np.allclose(whole.frequencies(), 2000.0 ** (-np.arange(16) / 16.0), rtol=1e-6)
    # no rotation at all: nothing to look up
    assert model_of(CFG_C).blocks[0].mixer.mixers[0].position.rotary_tables() is None


def test_what_the_config_leaves_out_does_not_exist():
    m = model_of(CFG_A)
    assert m.blocks[2].ffn is None and m.blocks[3].ffn is None and m.blocks[0].ffn is not None
    names = {r.name for r in m.tensor_reqs()}
    assert "l2.norm2" not in names and not any(n.startswith("l2.mlp") for n in names)
    assert isinstance(m.blocks[0].entry_norm(), tuple) and not isinstance(m.blocks[2].entry_norm(), tuple)
    c = model_of(CFG_C)
    assert c.blocks[2].mixer.mixers[0].chunk == 0 and c.blocks[0].mixer.mixers[0].chunk == 5
    assert [b.mult for b in c.blocks] == [0.25] * 3 and [b.mult for b in model_of(CFG_B).blocks] == [1.0] * 3
    assert tuple(model_of(CFG_B).blocks[2].mixer.spec.scales) == (0.5, 2.0)


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="conv"), "unknown type"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "multiple of kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(tau=0.0), "tau"),
    (lambda c: c["layers"][0]["mixer"].pop("right"), "right"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "mlp.kind"),
    (lambda c: c["layers"][1]["mixer"].update(state=500), "state"),
    (lambda c: c["layers"][1]["mixer"].pop("conv"), "conv"),
])
def test_a_config_that_cannot_be_served_says_why(change, message):
    cfg = copy.deepcopy(CFG_A)
    change(cfg)
    with pytest.raises(ConfigError) as e:
        resolve_architecture(cfg).config_from_dict(cfg)
    assert message in str(e.value)


# ---------------------------------------------------------------- the plain implementation against closed forms
def test_plain_chunk_mask_edges():
    seen = P.chunk_mask(np.arange(10), 4)
    assert seen[3, 0] and seen[3, 3] and not seen[4, 3] and seen[4, 4] and seen[7, 4] and not seen[8, 7] and not seen[2, 3]
    shifted = P.chunk_mask(np.arange(6, 10), 4)          # chunks are counted from position 0
    assert shifted[1, 0] and not shifted[2, 1] and shifted[3, 2]
    assert P.chunk_mask(np.arange(5), None).sum() == 15


def test_plain_sink_softmax_sums_to_less_than_one():
    rng = np.random.default_rng(0)
    q, k = rng.normal(size=(5, 2, 4)), rng.normal(size=(5, 1, 4))
    v = np.ones((5, 1, 3))
    o = P.sink_softmax_attention(q, k, v, 0.7, P.chunk_mask(np.arange(5), None), np.float64)
    for h in range(2):
        for t in range(5):
            e = np.exp((k[:t + 1, 0] @ q[t, h]) * 0.7)
            assert abs(o[t, h, 0] - e.sum() / (1.0 + e.sum())) < 1e-12
    full = P.sink_softmax_attention(q, k, v, 0.7, P.chunk_mask(np.arange(5), None), np.float64, sink=False)
    assert np.allclose(full, 1.0)


def test_plain_rotation_pairs_i_with_i_plus_half_and_leaves_the_rest():
    x = np.zeros((1, 1, 8))
    x[0, 0, 1] = 1.0
    x[0, 0, 6] = 5.0
    f = P.rotary_frequencies(4, 100.0, 2.0)
    assert np.allclose(f, [0.5, 0.05])
    y = P.rotate_half(x, np.array([3]), f, np.float64)[0, 0]
    assert np.allclose(y[[1, 3]], [np.cos(0.15), np.sin(0.15)]) and y[6] == 5.0 and y[0] == 0 and y[2] == 0


def test_plain_decayed_outer_products_closed_form():
    """Constant decays: o_t = sum_j (q . (alpha^(t - j) k_j)) v_j."""
    rng = np.random.default_rng(1)
    T, H, D, E = 6, 2, 3, 4
    q, k, v = rng.normal(size=(T, H, D)), rng.normal(size=(T, H, D)), rng.normal(size=(T, H, E))
    a = rng.uniform(0.3, 0.9, (H, D))
    o = P.decayed_outer_products(q, k, v, np.tile(a[None], (T, 1, 1)), np.float64)
    for t in range(T):
        for h in range(H):
            want = sum(((q[t, h] * a[h] ** (t - j)) @ k[j, h]) * v[j, h] for j in range(t + 1))
            assert np.allclose(o[t, h], want)


def test_plain_selective_scan_closed_form():
    """A constant step: S_t = sum_j exp(d A)^(t - j) d x_j B_j."""
    rng = np.random.default_rng(2)
    T, I, N = 5, 3, 2
    x, B, C = rng.normal(size=(T, I)), rng.normal(size=(T, N)), rng.normal(size=(T, N))
    A, D = -rng.uniform(0.1, 1.0, (I, N)), rng.normal(size=I)
    d = np.full((T, I), 0.4)
    y = P.selective_scan(x, d, A, B, C, D, np.float64)
    for t in range(T):
        S = sum(np.exp(0.4 * A) ** (t - j) * 0.4 * x[j][:, None] * B[j][None] for j in range(t + 1))
        assert np.allclose(y[t], S @ C[t] + D * x[t])


def test_plain_convolution_reads_zeros_before_the_start_and_the_last_tap_is_now():
    x = np.arange(1.0, 5.0)[:, None]
    w = np.array([[100.0, 10.0, 1.0]])
    y = P.causal_conv(x, w, np.array([0.5]), np.float64)[:, 0]
    assert list(y) == [1.5, 12.5, 123.5, 234.5]


def test_plain_prefix_property_and_float32_agrees():
    from bumolix_util import random_weights
    for cfg, seed in ((CFG_A, 1), (CFG_C, 2)):
        w = random_weights(cfg, seed)
        toks = np.random.default_rng(seed).integers(0, cfg["vocab"], 40).tolist()
        z = P.forward(cfg, w, toks, np.float64)
        assert np.allclose(P.forward(cfg, w, toks[:17], np.float64), z[:17], atol=1e-10)
        assert np.abs(P.forward(cfg, w, toks, np.float32) - z).max() < 2e-4 * np.abs(z).max()


def test_plain_layer_reads_two_norms_of_the_same_stream():
    """h + m (mixer(norm1 h) + ffn(norm2 h)): swapping the gains changes the result, scaling m scales the step."""
    from bumolix_util import random_weights
    cfg = config([parallel_layer(mlp=dense(24))], vocab=30, width=32, mult=0.5)
    w = random_weights(cfg, 3)
    h = np.random.default_rng(3).normal(size=(7, 32))
    pos = np.arange(7)
    step = P.layer(h, pos, w, 0, cfg, np.float64) - h
    twice = dict(cfg, residual_mult=1.0)
    assert np.allclose(P.layer(h, pos, w, 0, twice, np.float64) - h, 2 * step)
    swapped = dict(w)
    swapped["l0.norm1"], swapped["l0.norm2"] = w["l0.norm2"], w["l0.norm1"]
    assert np.abs(P.layer(h, pos, swapped, 0, cfg, np.float64) - h - step).max() > 1e-3
