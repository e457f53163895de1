"""Buketar on the CPU: config.json -> specification (run order, tensors, constants), the rotation law's
frequencies against the plain implementation's, errors that name the key, and the plain implementation's own
consistency (a prefix's logits do not depend on what follows; a loop is the same as its layers written out; one
stream with unit connections is the ordinary residual sum)."""
import copy

import numpy as np
import pytest
import torch

import plain_buketar as pb
from buketar_configs import CONFIGS, random_tokens, random_weights, tensor_shapes


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_spec_lists_the_designs_tensors(name):
    from inferrs_amd.config.buketar import BuketarConfig
    from inferrs_amd.config.registry import resolve_architecture
    from inferrs_amd.parts.assemble import model_tensors
    cfg = CONFIGS[name]
    assert resolve_architecture(cfg) is BuketarConfig
    spec = BuketarConfig.from_dict(cfg).to_spec()
    expected, optional = model_tensors(spec)
    want = tensor_shapes(cfg)
    assert set(expected) == set(want)
    assert {k: tuple(v.shape) for k, v in expected.items()} == want
    assert [e.layer for e in spec.schedule] == pb.run_order(cfg)
    assert all(e.cache_of is None for e in spec.schedule)          # every pass of a looped layer owns its cache or state
    assert BuketarConfig.from_dict(cfg).to_dict() == cfg


def test_constants_come_from_the_config():
    from inferrs_amd.config.buketar import BuketarConfig
    spec = BuketarConfig.from_dict(CONFIGS["A"]).to_spec()
    att, rec = spec.layers[1].mixer, spec.layers[0].mixer
    assert (att.n_heads, att.head_dim, att.rot_dim, att.v_dim, att.kv_rank, att.scale) == (3, 24, 8, 20, 40, 0.2)
    assert att.position.rot_dim == 4 and att.position.theta == 5000.0 and att.position.scaling == ("yarn", 4.0, 64.0, 8.0, 1.0)
    assert att.norm_eps == 1e-5 and spec.final_norm.eps == 1e-5
    assert (rec.width, rec.blocks, rec.conv, rec.decay) == (40, 2, 4, 8.0)
    ffn = spec.layers[3].ffn
    assert (ffn.intermediate, ffn.experts, ffn.top, ffn.scale, ffn.limit, ffn.alpha) == (16, 3, 3, 0.7, 0.5, 1.702)
    assert spec.layers[2].ffn is None and len(spec.layers[2].norms) == 1
    assert spec.head.cap == 12.0 and spec.layers[0].residual.streams == 2 and spec.layers[0].residual.connections
    plain = BuketarConfig.from_dict(CONFIGS["B"]).to_spec()
    assert plain.head.cap is None and not plain.layers[0].residual.connections and plain.layers[0].residual.streams == 1
    assert plain.layers[0].mixer.position.scaling is None


@pytest.mark.parametrize("change, key", [
    (lambda c: c["layers"][0].update(type="conv"), "layers[0].type"),
    (lambda c: c["layers"][0]["mixer"].update(width=41), "layers[0].mixer.width"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "router.top"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "layers[1].mixer.kv_rank"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["loop"].update(stop=7), "loop"),
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "mlp.kind"),
])
def test_a_bad_config_names_its_key(change, key):
    from inferrs_amd.config.base import ConfigError
    from inferrs_amd.config.buketar import BuketarConfig
    cfg = copy.deepcopy(CONFIGS["A"])
    change(cfg)
    with pytest.raises(ConfigError, match=key.replace("[", r"\[").replace("]", r"\]")):
        BuketarConfig.from_dict(cfg)


@pytest.mark.parametrize("rot", [
    {"base": 5000.0, "dims": 4, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0, "slow": 1.0}},
    {"base": 100.0, "dims": 32, "scaling": {"factor": 16.0, "original": 32, "fast": 4.0, "slow": 2.0}},
    {"base": 500000.0, "dims": 64, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
    {"base": 10000.0, "dims": 6, "scaling": None},
])
def test_rotation_frequencies_follow_the_law(rot):
    from inferrs_amd.config.spec import PositionSpec
    from inferrs_amd.parts.base import part_class
    sc = rot["scaling"]
    spec = PositionSpec("rope", head_dim=rot["dims"], rot_dim=rot["dims"], theta=rot["base"], pairing="half",
                        scaling=("yarn", sc["factor"], sc["original"], sc["fast"], sc["slow"]) if sc else None)
    part = part_class("position", spec)(spec, {}, torch.float32, "cpu")
    f, m = pb.rotary_frequencies(rot)
    np.testing.assert_allclose(part.inv_freq.numpy(), f.numpy(), rtol=2e-6)
    assert abs(part.magnitude - m) < 1e-12
    if sc:
        assert part.magnitude > 1.0 and (f.numpy() <= np.array([rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)]) * (1 + 1e-12)).all()


def test_plain_prefix_loop_and_single_stream():
    cfg = CONFIGS["A"]
    w = random_weights(cfg, 1)
    toks = random_tokens(30, cfg["vocab"], 2)
    full = pb.forward(cfg, w, toks)
    np.testing.assert_allclose(pb.forward(cfg, w, toks[:11]).numpy(), full[:11].numpy(), atol=1e-10)
    # the loop written out: layers 1, 2 twice in a row
    flat = copy.deepcopy(cfg)
    del flat["loop"]
    order = pb.run_order(cfg)
    flat["layers"] = [cfg["layers"][i] for i in order]
    w2 = {}
    for name, t in w.items():
        if not name.startswith("l"):
            w2[name] = t
    for new, old in enumerate(order):
        for name, t in w.items():
            if name.startswith(f"l{old}."):
                w2[f"l{new}." + name.split(".", 1)[1]] = t
    np.testing.assert_allclose(pb.forward(flat, w2, toks).numpy(), full.numpy(), atol=1e-10)
    # one stream whose connections are all 1 is the plain residual sum
    one = copy.deepcopy(CONFIGS["B"])
    wb = random_weights(one, 3)
    short = random_tokens(9, one["vocab"], 4)
    plain = pb.forward(one, wb, short)
    one["streams"] = 1
    for i, L in enumerate(one["layers"]):
        for q in ([1] if L["mlp"] is None else [1, 2]):
            wb[f"l{i}.hc{q}.in"] = torch.ones(1)
            wb[f"l{i}.hc{q}.out"] = torch.ones(1)
            wb[f"l{i}.hc{q}.mix"] = torch.ones(1, 1)
    np.testing.assert_allclose(pb.forward(one, wb, short).numpy(), plain.numpy(), atol=1e-10)
