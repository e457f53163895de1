"""Random Buketar configurations through the engine against the plain implementation: layer orders, loops, stream
counts (or none), head counts, cached rows in and out of the sizes the matrix-core attention takes (16 to 256 in steps
of 16), partly rotated features with and without the scaling law, value sizes other than key sizes, recurrences of 1 to
5 taps in 1 to 4 blocks, 2 to 12 experts of which 1 to all run, widths from odd ones to those whose products run on the
kernels for many rows, vocabularies of any size.  Every configuration runs whole prompts and a mixed schedule (four live
requests, pages and slots used again) in 32-bit (2e-5 of the largest logit at every position) and in bfloat16 (the
distribution of the errors against the plain implementation's in bfloat16 arithmetic, as in `test_buketar_gpu.py`)."""
import io
import random

import numpy as np
import pytest
import torch

import plain_buketar as pb
import trace_modes as tm
from buketar_configs import attention, layer, moe, random_tokens, recurrence, write_model

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 19, 64, 130, 260]


def random_config(rng: random.Random) -> dict:
    big = rng.random() < 0.35
    width = rng.choice([128, 256, 384]) if big else rng.choice([24, 33, 40, 50, 64, 72, 96])
    n_layers = rng.randint(1, 4)
    layers = []
    for _ in range(n_layers):
        ff = rng.choice([64, 128]) if big else rng.choice([10, 16, 24, 30, 40])
        experts = rng.randint(2, 12)
        mlp = None if rng.random() < 0.2 else moe(ff, experts, rng.randint(1, experts), rng.choice([0.5, 1.0, 2.0, 2.5]),
                                                  rng.choice([0.5, 1.0, 3.0, 7.0]))
        if rng.random() < 0.5:
            rot_dim = rng.choice([2, 4, 6, 8, 16, 32])
            rank = rng.choice([16 - rot_dim, 32 - rot_dim, 48 - rot_dim, 64 - rot_dim, 112 - rot_dim, 128 - rot_dim, 224 - rot_dim,
                               20, 27, 50, 90]) if rng.random() < 0.7 else rng.randint(4, 120)
            rank = max(rank, 4)
            turned = rng.choice([rot_dim, rot_dim, max(2, rot_dim // 2 // 2 * 2)])
            scaling = None if rng.random() < 0.4 else {"factor": rng.choice([2.0, 8.0, 40.0]), "original": rng.choice([16, 64, 1024]),
                                                       "fast": rng.choice([4.0, 32.0]), "slow": rng.choice([1.0, 2.0])}
            mixer = attention(rng.randint(1, 12), rng.choice([8, 12, 16, 24, 64]), rot_dim, rng.choice([8, 10, 16, 32, 64]), rank,
                              rng.choice([0.05, 0.1, 0.2]), base=rng.choice([100.0, 10000.0, 500000.0]), turned=turned, scaling=scaling)
        else:
            blocks = rng.randint(1, 4)
            per = rng.choice([32, 64, 128]) if big else rng.choice([5, 8, 14, 16, 20])
            mixer = recurrence(blocks * per, blocks, rng.randint(1, 5))
        layers.append(layer(mixer, mlp))
    cfg = {"architecture": "Buketar", "vocab": rng.choice([31, 64, 100, 257, 576]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.8:
        cfg["streams"] = rng.randint(1, 4)
    if rng.random() < 0.7:
        cfg["logit_softcap"] = rng.choice([10.0, 30.0, 50.0])
    if rng.random() < 0.6:
        start = rng.randint(0, n_layers - 1)
        cfg["loop"] = {"start": start, "stop": rng.randint(start, n_layers), "times": rng.randint(1, 3)}
    return cfg


def run(folder, cfg, dtype, trace, out_dir):
    from inferrs_amd.engine import Engine, run_trace
    eng = Engine.from_folder(folder, dtype=dtype, page_size=16, num_pages=-(-trace.max_tokens // 16), max_seqs=4)
    run_trace(eng, trace.lines, out_dir, io.StringIO())
    eng.cache.check_invariants()
    assert not eng.cache.sequences and eng.cache.slots.num_free == eng.cache.slots.num_slots
    return trace.read(out_dir, cfg["vocab"])


def errors(got, ref, reqs):
    scale = max(float(np.abs(v).max()) for v in ref.values())
    return np.concatenate([[float(np.abs(got[r][p] - ref[r][p]).max()) / scale for p in range(len(t))] for r, t in reqs.items()])


@pytest.mark.parametrize("seed", range(20))
def test_random_configuration(tmp_path, seed):
    rng = random.Random(4000 + seed)
    cfg = random_config(rng)
    folder = write_model(str(tmp_path / "model"), cfg, seed=seed, sharpen=rng.choice([1.0, 1.0, 3.0]))
    _, tensors = pb.load_folder(folder)
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate(LENGTHS)}
    ref = {r: pb.forward(cfg, tensors, t).numpy().astype(np.float32) for r, t in reqs.items()}
    rounded = {r: pb.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in reqs.items()}
    theirs = errors(rounded, ref, reqs)
    for mode, trace in (("whole", tm.whole(reqs)), ("mixed", tm.mixed(reqs, seed=seed))):
        got = run(folder, cfg, "float32", trace, str(tmp_path / f"{mode}_f32"))
        err = errors(got, ref, reqs)
        assert err.max() <= 2e-5, f"seed {seed} {mode} float32: {err.max():.3g} of the scale; {cfg}"
        got = run(folder, cfg, "bfloat16", trace, str(tmp_path / f"{mode}_bf16"))
        mine = errors(got, ref, reqs)
        assert np.isfinite(mine).all(), f"seed {seed} {mode} bfloat16: not finite; {cfg}"
        for q, slack in ((0.5, 1.1), (0.9, 1.5)):
            a, b = float(np.quantile(mine, q)), float(np.quantile(theirs, q))
            assert a <= slack * b + 1e-3, f"seed {seed} {mode} bfloat16: quantile {q} of the errors {a:.3g}, plain in bfloat16 {b:.3g}; {cfg}"
