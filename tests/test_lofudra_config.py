"""Lofudra without a GPU: config.json -> the model as data (layers, run order, tensor names and shapes, what each
mixer keeps per request), the errors that name a key, the cache manager with a mixer that keeps pages and a state, and
the plain implementation against itself (a loop of one pass, a window wider than the sequence, whole against prefix)."""
import copy

import pytest
import torch

import plain_lofudra as pl
from lofudra_configs import CONFIGS, random_tokens, random_weights, tensor_shapes

from inferrs_amd.cache import CacheManager
from inferrs_amd.config.base import ConfigError
from inferrs_amd.config.lofudra import LofudraConfig
from inferrs_amd.config.registry import resolve_architecture
from inferrs_amd.parts.assemble import model_tensors
from inferrs_amd.parts.base import FixedState, PagedAndState, PagedKV, part_class


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_tensor_names_and_shapes(name):
    cfg = CONFIGS[name]
    assert resolve_architecture(cfg) is LofudraConfig
    spec = LofudraConfig.from_dict(cfg).to_spec()
    expected, optional = model_tensors(spec)
    assert {k: tuple(v.shape) for k, v in expected.items()} == tensor_shapes(cfg)
    assert not optional - set(expected)


def test_run_order_marks_the_passes():
    spec = LofudraConfig.from_dict(CONFIGS["A"]).to_spec()
    assert [(e.layer, e.pass_index) for e in spec.schedule] == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (3, None)]
    assert spec.pass_input.times == 2 and spec.pass_input.name == "loop.step"
    spec = LofudraConfig.from_dict(CONFIGS["C"]).to_spec()
    assert [(e.layer, e.pass_index) for e in spec.schedule] == [(0, 0), (1, None), (0, 1), (1, None), (0, 2), (1, None)]
    spec = LofudraConfig.from_dict(CONFIGS["B"]).to_spec()
    assert [e.layer for e in spec.schedule] == [0, 1, 2] and spec.pass_input is None
    assert [len(l.norms) for l in spec.layers] == [4, 4, 2]


def test_what_each_mixer_keeps():
    spec = LofudraConfig.from_dict(CONFIGS["A"]).to_spec()
    needs = [part_class("mixer", l.mixer).cache_need(l.mixer) for l in spec.layers]
    assert needs[0] == FixedState((3 * 8 * 16 + 2 * (3 * 8 + 2 * 16),), torch.float32)
    assert needs[1] == PagedAndState(PagedKV(2, 16, 24), FixedState((2 * 24 * 8,), torch.float32))
    assert needs[2] == FixedState((2 * 17 * 24 + 2,), torch.float32)
    left = spec.layers[1].mixer.left
    assert left.sink and left.values_from_keys and left.qkv_bias and left.window == 24 and left.position.rot_dim == 8
    no_window = LofudraConfig.from_dict(CONFIGS["D"]).to_spec().layers[0].mixer.left
    assert no_window.window is None and no_window.position.kind == "none"


def test_pages_and_a_state_for_one_layer():
    spec = LofudraConfig.from_dict(CONFIGS["A"]).to_spec()
    needs = {}
    for stop, e in enumerate(spec.schedule):
        m = spec.layers[e.layer].mixer
        needs[stop] = part_class("mixer", m).cache_need(m)
    cm = CacheManager(needs, page_size=8, num_pages=10, max_seqs=2)
    assert len(cm.groups) == 1 and cm.groups[0].layers == [1, 3, 5] and cm.groups[0].need.window == 24
    assert sorted(st.layer for st in cm.states) == [0, 1, 2, 3, 4, 5]
    a = cm.add_sequence("a")
    assert cm.reserve("a", 30)
    cm.commit("a", 30)
    cm.free_sequence("a")
    cm.check_invariants()
    assert cm.groups[0].pool.num_free == 10 and cm.slots.num_free == 2


@pytest.mark.parametrize("change, key", [
    (lambda c: c["layers"][1].__setitem__("type", "attention"), "layers[1].type"),
    (lambda c: c["layers"][1]["mixer"]["left"].__setitem__("vdim", 8), "vdim"),
    (lambda c: c["layers"][1]["mixer"]["right"].__setitem__("decay", [0.5]), "decay"),
    (lambda c: c["layers"][1]["mixer"]["left"].pop("scale"), "left.scale"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("groups", 2), "groups"),
    (lambda c: c["layers"][0]["mixer"].__setitem__("norm_groups", 5), "norm_groups"),
    (lambda c: c["layers"][2]["mixer"].pop("gate_cap"), "gate_cap"),
    (lambda c: c["layers"][0]["mlp"].__setitem__("kind", "moe"), "mlp.kind"),
    (lambda c: c["loop"].__setitem__("stop", 9), "loop"),
    (lambda c: c["norm"].pop("eps"), "norm.eps"),
    (lambda c: c.pop("width"), "width"),
])
def test_errors_name_the_key(change, key):
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError) as e:
        LofudraConfig.from_dict(cfg)
    assert key in str(e.value)


def test_plain_against_itself():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 3)
    toks = random_tokens(60, cfg["vocab"], 1)
    whole = pl.forward(cfg, w, toks)
    # causal: a prefix gives the same logits
    assert torch.allclose(pl.forward(cfg, w, toks[:23]), whole[:23], atol=1e-10)
    # a window wider than the sequence is no window
    wide, none = copy.deepcopy(cfg), copy.deepcopy(cfg)
    for L in wide["layers"]:
        if L["type"] == "parallel":
            L["mixer"]["left"]["mask"]["size"] = 1000
    for L in none["layers"]:
        if L["type"] == "parallel":
            L["mixer"]["left"].pop("mask")
    assert torch.equal(pl.forward(wide, w, toks), pl.forward(none, w, toks))
    assert not torch.allclose(pl.forward(wide, w, toks), whole, atol=1e-3)
    # the stream after every layer run: one entry a stop of the run order
    trace = []
    pl.forward(cfg, w, toks, trace=trace)
    assert len(trace) == 6
