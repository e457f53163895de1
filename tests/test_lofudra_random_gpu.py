"""Random Lofudra configurations through the engine against the plain implementation: layer orders, loops (from layer
0, of one pass, over everything, none), layers without feed-forward, query and key head counts, head sizes in and out of
those the matrix-core attention takes (16 to 256 in steps of 16) and the fused decode kernel (steps of 64), windows from
1 to longer than any request or none, whole heads rotating, parts of them or nothing, retention decays from 0 to 1,
matrix memories and state spaces whose key and value sizes fit no vector width, 1 to 6 taps, grouped B and C, norm
groups, widths from odd ones to those whose products run on the kernels for many rows, vocabularies of any size.  Every
configuration runs whole prompts, a prompt and then token by token, and a mixed schedule (four live requests, pages and
slots used again) in 32-bit (2e-5 of the largest logit at every position, or three times what the plain implementation's
own 32-bit arithmetic is off there) and in bfloat16 (the distribution of the errors against the plain implementation's in
bfloat16 arithmetic, as in `test_lofudra_gpu.py`)."""
import io
import random

import numpy as np
import pytest
import torch

import plain_lofudra as pl
import trace_modes as tm
from lofudra_configs import layer, left, mamba2, mlstm, parallel, random_tokens, right, write_model

pytestmark = pytest.mark.gpu

LENGTHS = [1, 2, 19, 64, 150, 260]


def random_mixer(rng: random.Random, big: bool):
    kind = rng.choice(["parallel", "mlstm", "mamba2"])
    if kind == "parallel":
        kv = rng.choice([1, 1, 2, 3])
        dim = rng.choice([16, 32, 64, 128]) if rng.random() < 0.6 else rng.choice([8, 12, 24, 40, 80, 96])
        turned = rng.choice([dim, dim, dim // 2 // 2 * 2, 0])
        heads_r = rng.randint(1, 4)
        return parallel(left(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([0.05, 0.125, 0.3]),
                             window=rng.choice([None, 1, 7, 16, 33, 64, 100, 1000]), base=rng.choice([100.0, 10000.0, 500000.0]),
                             turned=turned),
                        right(heads_r, rng.choice([4, 8, 10, 32, 64] if not big else [32, 64, 128]), rng.choice([4, 6, 16, 24, 64]),
                              [rng.choice([0.0, 0.5, 0.9, 0.97, 0.999, 1.0]) for _ in range(heads_r)]),
                        rng.choice([0.5, 1.0, 1.7]), rng.choice([0.3, 1.0, 2.0]))
    if kind == "mlstm":
        return mlstm(rng.randint(1, 4), rng.choice([8, 10, 24, 48, 64] if not big else [64, 128]), rng.choice([6, 8, 16, 33, 48]),
                     rng.choice([4.0, 10.0, 15.0]))
    groups = rng.choice([1, 1, 2, 3])
    heads = groups * rng.randint(1, 3)
    vdim = rng.choice([4, 6, 8, 16, 32])
    parts = rng.choice([p for p in (1, 2, 3, 4, heads) if (heads * vdim) % p == 0])
    return mamba2(heads, vdim, rng.choice([8, 12, 16, 48, 64] if not big else [64, 128]), groups, rng.randint(1, 6), parts)


def random_config(rng: random.Random) -> dict:
    big = rng.random() < 0.35
    width = rng.choice([128, 256, 384]) if big else rng.choice([24, 33, 40, 50, 64, 72, 96])
    n_layers = rng.randint(1, 4)
    layers = [layer(random_mixer(rng, big), None if rng.random() < 0.2 else (rng.choice([64, 128, 512]) if big else rng.choice([10, 16, 24, 40])))
              for _ in range(n_layers)]
    cfg = {"architecture": "Lofudra", "vocab": rng.choice([31, 64, 100, 257, 576]), "width": width,
           "norm": {"eps": rng.choice([1e-6, 1e-5])}, "layers": layers}
    if rng.random() < 0.7:
        start = rng.randint(0, n_layers - 1)
        cfg["loop"] = {"start": start, "stop": rng.randint(start + 1, n_layers), "times": rng.randint(1, 3)}
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


@pytest.mark.parametrize("seed", range(24))
def test_random_configuration(tmp_path, seed):
    rng = random.Random(7000 + seed)
    cfg = random_config(rng)
    tensors = write_model(str(tmp_path / "model"), cfg, seed=seed, sharpen=rng.choice([1.0, 1.0, 4.0]))
    folder = str(tmp_path / "model")
    reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 70 + i) for i, n in enumerate(LENGTHS)}
    ref64 = {r: pl.forward(cfg, tensors, t) for r, t in reqs.items()}
    ref = {r: v.numpy().astype(np.float32) for r, v in ref64.items()}
    noise = errors({r: pl.forward(cfg, tensors, t, dtype=torch.float32).double().numpy() for r, t in reqs.items()},
                   {r: v.numpy() for r, v in ref64.items()}, reqs)
    rounded = {r: pl.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in reqs.items()}
    theirs = errors(rounded, ref, reqs)
    for mode, trace in (("whole", tm.whole(reqs)), ("tail", tm.prefix_then_single(reqs, 40)), ("mixed", tm.mixed(reqs, seed=seed))):
        got = run(folder, cfg, "float32", trace, str(tmp_path / f"{mode}_f32"))
        err = errors(got, ref, reqs)
        assert (err <= np.maximum(2e-5, 3.0 * noise)).all(), \
            f"seed {seed} {mode} float32: {err.max():.3g} of the scale (the plain 32-bit arithmetic: {noise.max():.3g}); {cfg}"
        got = run(folder, cfg, "bfloat16", trace, str(tmp_path / f"{mode}_bf16"))
        mine = errors(got, ref, reqs)
        assert np.isfinite(mine).all(), f"seed {seed} {mode} bfloat16: not finite; {cfg}"
        for q, slack in ((0.5, 1.1), (0.9, 1.5)):
            a, b = float(np.quantile(mine, q)), float(np.quantile(theirs, q))
            assert a <= slack * b + 1e-3, f"seed {seed} {mode} bfloat16: quantile {q} of the errors {a:.3g}, plain in bfloat16 {b:.3g}; {cfg}"
