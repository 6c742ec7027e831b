"""Rotalorn on the host: the registry, config.json's keys, the tensor list, what a request keeps,
the scaled frequencies, the plain mechanisms against cases made by hand, error messages."""
import copy
import math

import numpy as np
import pytest

from plain import rotalorn_plain as P
from rotalorn_util import (CFG_A, CFG_B, CFG_C, attention_layer, config, dense, diff_layer, latent_layer, moe,
                           tensor_shapes)
from zse_amd import models as _models  # noqa: F401
from zse_amd.config.base import ConfigError, resolve_architecture
from zse_amd.config.plan import RotarySpec
from zse_amd.engine.model import Model
from zse_amd.parts.base import PagedKV
from zse_amd.parts.position import Rotary


def model_of(cfg):
    arch = resolve_architecture(cfg)
    return Model(arch.plan(arch.config_from_dict(cfg)))


def test_the_architecture_is_found_by_its_name():
    assert resolve_architecture(CFG_A).name == "Rotalorn"
    assert resolve_architecture({"model_type": "rotalorn"}).name == "Rotalorn"


@pytest.mark.parametrize("cfg", [CFG_A, CFG_B, CFG_C])
def test_the_tensor_list_is_the_checkpoints(cfg):
    reqs = {r.name: tuple(r.shape) for r in model_of(cfg).tensor_reqs()}
    assert reqs == tensor_shapes(cfg)


def test_what_a_request_keeps():
    m = model_of(CFG_A)
    needs = m.cache_needs()
    assert all(isinstance(n, PagedKV) for n in needs)
    latent, diff, attn, diff2 = needs
    assert (latent.num_kv_heads, latent.head_dim, latent.window, latent.values_in_keys) == (1, 24, 13, True)
    assert (diff.num_kv_heads, diff.head_dim, diff.value_heads, diff.value_dim, diff.window) == (4, 12, 2, 24, None)   # a key head a map
    assert (attn.num_kv_heads, attn.head_dim, attn.window) == (2, 24, 21)
    assert (diff2.num_kv_heads, diff2.head_dim, diff2.value_heads, diff2.value_dim) == (4, 8, 2, 8)
    assert m.embedding.state_bytes() == 4                     # the previous token
    assert model_of(CFG_B).embedding.state_bytes() == 0       # no pair table, nothing kept
    assert model_of(CFG_B).cache_needs()[1].window is None and model_of(CFG_B).cache_needs()[3].window is None


def test_every_constant_comes_from_the_config():
    arch = resolve_architecture(CFG_A)
    plan = arch.plan(arch.config_from_dict(CFG_A))
    d = plan.layers[1].mixer
    assert (d.diff, d.softcap, d.temp_coef, d.temp_every, d.scale) == (0.4, 15.0, 0.5, 16, 12 ** -0.5)
    assert plan.layers[3].mixer.softcap is None and plan.layers[3].mixer.temp_every == 5
    a = plan.layers[2].mixer
    assert a.values_are_keys and a.scale == 0.3 and a.position.wavelength_scaling == (6.0, 1.0, 3.0, 64.0)
    assert a.position.rotary_dim == 12 and a.norm_eps == 1e-5
    f = plan.layers[1].ffn
    assert (f.scoring, f.scale_input, f.activation, f.top_k, f.num_experts) == ("softmax", False, "silu", 2, 5)
    assert f.shared_gate == "l1.mlp.shared.sg" and plan.layers[0].ffn.activation == "gelu_tanh"
    assert plan.embedding.pairs.buckets == 61 and (plan.embedding.pairs.mul_prev, plan.embedding.pairs.mul_cur) == (7, 3)
    assert plan.head.weight == plan.embedding.weight          # the logits come from the embedding table
    b = arch.plan(arch.config_from_dict(CFG_B))
    assert b.layers[2].mixer.temp_every == 0 and b.layers[2].mixer.softcap is None and b.embedding.pairs is None
    assert b.layers[1].ffn is None and b.layers[0].ffn.shared is None and b.layers[0].ffn.shared_gate is None


@pytest.mark.parametrize("dims,base,scaling", [(12, 500.0, (6.0, 1.0, 3.0, 64)), (16, 50.0, (4.0, 1.0, 2.0, 32)),
                                               (4, 10.0, (2.0, 1.0, 4.0, 16)), (64, 5e5, (6.0, 1.0, 3.0, 512)),
                                               (32, 1e4, None)])
def test_frequencies_scaled_by_their_wavelengths(dims, base, scaling):
    part = Rotary(RotarySpec(head_dim=dims, rotary_dim=dims, theta=base, wavelength_scaling=scaling))
    want = P.rotary_frequencies(dims, base, dict(zip(("factor", "low", "high", "original"), scaling)) if scaling else None)
    assert np.allclose(part.frequencies(), want.astype(np.float32), rtol=1e-6, atol=0)
    if scaling:
        factor, low, high, orig = scaling
        plain = np.array([base ** (-2.0 * i / dims) for i in range(dims // 2)])
        lengths = 2 * math.pi / plain
        assert np.allclose(want[lengths < orig / high], plain[lengths < orig / high])
        assert np.allclose(want[lengths > orig / low], plain[lengths > orig / low] / factor)
        mid = (lengths >= orig / high) & (lengths <= orig / low)
        assert np.all(want[mid] <= plain[mid] * (1 + 1e-12)) and np.all(want[mid] >= plain[mid] / factor * (1 - 1e-12))


def test_plain_mechanisms_against_cases_made_by_hand():
    assert P.bigram_rows([5, 9, 2], 11, 7, 3).tolist() == [11, (5 * 7 + 9 * 3) % 11, (9 * 7 + 2 * 3) % 11]
    assert P.bigram_rows([4], 1, 1, 1).tolist() == [1]
    t = P.query_temperature([0, 14, 15, 16, 47], 0.5, 16, np.float64)
    assert np.allclose(t, [1.0, 1.0, 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(2), 1 + 0.5 * math.log(4)])
    w = {"a.lq1": np.array([1.0, 2.0]), "a.lk1": np.array([0.5, 0.25]), "a.lq2": np.array([0.0, 1.0]), "a.lk2": np.array([3.0, -1.0])}
    assert math.isclose(P.differential_lambda(w, "a.", 0.3), math.exp(1.0) - math.exp(-1.0) + 0.3)
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    y = P.layer_norm(x, np.array([2.0, 2.0, 2.0, 2.0]), np.array([0.5, 0.5, 0.5, 0.5]), 0.0, np.float64)
    assert np.allclose(y, (x - 3.0) / math.sqrt(3.5) * 2 + 0.5)
    ids, wts, margin = P.route(np.array([[1.0, 0.0]]), np.array([[0.0, 0.0], [2.0, 0.0], [1.0, 0.0], [2.0, 0.0]]), 2, np.float64)
    assert ids.tolist() == [[1, 3]]                         # the lower index among equals first
    e = np.exp([0.0, 2.0, 1.0, 2.0])
    assert np.allclose(wts, [[e[1] / e.sum(), e[3] / e.sum()]])        # scores of the softmax over all, not renormalised
    # a window of 3 sees itself and two tokens before it
    assert P.visible(5, 3)[4].tolist() == [False, False, True, True, True]
    # values that are keys: with one key the output is the key as projected, bias included, whatever norm and rotation do
    cfg = config([attention_layer(heads=1, kv_heads=1, dim=4, rot_dims=4, window=4)], vocab=8, width=4)
    ws = {"l0.mix.q": np.eye(4), "l0.mix.k": np.eye(4), "l0.mix.q.b": np.zeros(4), "l0.mix.k.b": np.array([1.0, 0, 0, 0]),
          "l0.mix.q.norm": np.ones(4), "l0.mix.k.norm": np.full(4, 9.0), "l0.mix.o": np.eye(4)}
    out = P.attention_mixer(cfg["layers"][0]["mixer"], ws, "l0.mix.", np.array([[0.5, 1.0, -1.0, 2.0]]), 1e-6, np.float64)
    assert np.allclose(out, [[1.5, 1.0, -1.0, 2.0]])


def test_errors_name_the_layer_and_the_key():
    bad = copy.deepcopy(CFG_A)
    bad["layers"][2]["mixer"]["vdim"] = 8
    bad["layers"][1]["mixer"].pop("diff")
    bad["layers"][0]["mixer"]["rot_dim"] = 3
    bad["layers"][3]["type"] = "conv"
    with pytest.raises(ConfigError) as e:
        resolve_architecture(bad).config_from_dict(bad)
    msg = str(e.value)
    assert "layer 2" in msg and "vdim" in msg and "layer 1" in msg and "'diff'" in msg and "layer 0" in msg and "rot_dim" in msg
    assert "layer 3" in msg and "conv" in msg
    for key in ("vocab", "width", "norm", "layers"):
        c = copy.deepcopy(CFG_B)
        c.pop(key)
        with pytest.raises(ConfigError, match=key):
            resolve_architecture(CFG_B).config_from_dict(c)
    c = copy.deepcopy(CFG_A)
    c["layers"][1]["mlp"]["router"]["top"] = 6
    with pytest.raises(ConfigError, match="top"):
        resolve_architecture(c).config_from_dict(c)
    c = copy.deepcopy(CFG_A)
    c["embedding"]["bigram"]["buckets"] = 0
    with pytest.raises(ConfigError, match="buckets"):
        resolve_architecture(c).config_from_dict(c)


def test_layers_of_other_kinds_can_be_put_together():
    cfg = config([diff_layer(mlp=None), latent_layer(mlp=moe(2, 1, 8, None)), attention_layer(mlp=dense(16))], width=24)
    m = model_of(cfg)
    assert [type(b.mixer).__name__ for b in m.blocks] == ["DifferentialAttention", "LatentAttention", "PagedAttention"]
    assert m.blocks[0].ffn is None
