"""Buketar on the GPU against the plain implementation (`plain_buketar.py`, 64-bit).

Mechanisms alone, through the kernels' Python face: the step between sub-layers over several residual streams,
the router with the experts, the convolution and the recurrence carried from portion to portion.  Then whole models
through the engine's step function under every way of cutting the work (whole prompts, a prompt and then token by
token, every token alone, portions down to two tokens, up to four live requests mixed in a pool whose pages and state
slots are used again), in both precisions, with ordinary weights and with sharpened queries (a query then singles
out a few keys somewhere in up to 700 tokens: at page borders, among the first tokens, far back).  Decays are drawn so
that some channels remember for hundreds of tokens: a state that is lost, not cleared or carried to the wrong request
shows.  Greedy generation runs through the engine's own entry point and scheduler.

Tolerances.  32-bit: 2e-5 of the largest logit against the 64-bit result, at every position.  bfloat16: rounding can
turn a router's close call, after which a position's logits are another model's, so single positions say little.  The
measure is the distribution of the positions' errors against that of the plain implementation in bfloat16 arithmetic
(every operation rounded) on the same positions: the engine keeps more in 32-bit than that, so its median and its
ninth decile must not be larger (a tenth and a half of slack)."""
import io
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_buketar as pb
import trace_modes as tm
from buketar_configs import CONFIGS, random_tokens, random_weights, write_model

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = [1, 2, 3, 17, 64, 65, 130, 300, 700]
TOL_F32 = 2e-5
CASES = [("A", 1.0), ("B", 1.0), ("C", 1.0), ("D", 1.0), ("E", 1.0), ("A", 4.0), ("B", 6.0), ("D", 4.0)]


def dev(t, dtype=None):
    return t.to(device="cuda", dtype=dtype or t.dtype).contiguous()


# ---- mechanisms alone ---------------------------------------------------------------------------

@pytest.mark.parametrize("S, W, K", [(1, 40, 1), (2, 33, 1), (3, 300, 4), (8, 64, 2)])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
def test_step_between_sublayers(S, W, K, y_dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(S * 100 + W)
    n = 19
    x = torch.randn(n, S, W, generator=g)
    y = torch.randn(n, K, W, generator=g).to(y_dtype)
    yw = torch.rand(n, K, generator=g) + 0.1
    ls, mix, out, read = torch.randn(W, generator=g), torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    nw = 1.0 + 0.1 * torch.randn(W, generator=g)
    xs = dev(x)
    if K == 1:
        h = ops.streams_step(xs, y=dev(y[:, 0]), scale=dev(ls), mix=dev(mix), out=dev(out), read=dev(read), norm_weight=dev(nw),
                             eps=1e-5, h_dtype=torch.float32)
    else:
        if y_dtype != torch.float32:
            pytest.skip("rows a chosen expert are 32-bit")
        h = ops.streams_step(xs, y=dev(y), y_weights=dev(yw), scale=dev(ls), mix=dev(mix), out=dev(out), read=dev(read),
                             norm_weight=dev(nw), eps=1e-5, h_dtype=torch.float32)
    yy = (y.double() * (yw.double()[:, :, None] if K > 1 else 1.0)).sum(1) * ls.double()
    new = torch.einsum("st,nsw->ntw", mix.double(), x.double()) + out.double()[None, :, None] * yy[:, None, :]
    np.testing.assert_allclose(xs.cpu().numpy(), new.numpy(), rtol=1e-5, atol=1e-5)
    u = torch.einsum("s,nsw->nw", read.double(), new)
    np.testing.assert_allclose(h.cpu().numpy(), pb.rms_norm(u, nw.double(), 1e-5).numpy(), rtol=1e-4, atol=1e-5)
    # a read of some rows with every stream counted once: the model's end
    rows = torch.tensor([5, 0, 18], dtype=torch.int32)
    tail = ops.streams_step(xs, rows=dev(rows), norm_weight=dev(nw), eps=1e-5, h_dtype=torch.float32)
    np.testing.assert_allclose(tail.cpu().numpy(), pb.rms_norm(new[rows.long()].sum(1), nw.double(), 1e-5).numpy(), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("E, top, W, ff, n", [(9, 1, 40, 20, 45), (5, 3, 33, 70, 45), (4, 4, 64, 16, 45), (70, 6, 48, 24, 45),
                                              (3, 2, 72, 200, 700)])
def test_router_and_experts(E, top, W, ff, n, dtype):
    """In 32-bit against the plain implementation; in bfloat16 (weights as tiles on the matrix cores where the sizes
    allow, few rows an expert and many) against the same with operands rounded as the kernels round them."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(E + top)
    lo = dtype == torch.bfloat16
    h = torch.randn(n, W, generator=g)
    w = {"router": 2.0 * torch.randn(E, W, generator=g) / W ** 0.5}
    for e in range(E):
        w[f"e{e}.gate"] = 1.5 * torch.randn(ff, W, generator=g) / W ** 0.5
        w[f"e{e}.up"] = 1.5 * torch.randn(ff, W, generator=g) / W ** 0.5
        w[f"e{e}.down"] = torch.randn(W, ff, generator=g) / ff ** 0.5
    if lo:
        h = h.bfloat16().float()
        w = {k: v.bfloat16().float() for k, v in w.items()}
    f = {"router": {"experts": E, "top": top, "scale": 1.7}, "expert": {"limit": 0.8}}
    want = pb.routed_experts(h.double(), {k: v.double() for k, v in w.items()}, f)
    gate_up = dev(torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) for e in range(E)]), dtype)
    down = dev(torch.stack([w[f"e{e}.down"] for e in range(E)]), dtype)
    tiled = ops.mix.experts_tiled_fits(dtype, W, ff)
    assert tiled == (lo and W % 8 == 0 and ff % 8 == 0)
    if tiled:
        gate_up, down = ops.mix.tile_weights(gate_up.view(E, 2, ff, W)), ops.mix.tile_weights(down)

    def run(rows):
        sel, weights = ops.route(dev(rows, dtype), dev(w["router"], dtype), top, 1.7)
        y = ops.experts_forward(dev(rows, dtype), sel, gate_up, down, 0.8, 1.702, ff=ff if tiled else None)
        return sel.cpu(), (y * weights[:, :, None]).sum(1).cpu(), y.cpu()

    sel, got, rows_all = run(h)
    s = torch.sigmoid(h.double() @ w["router"].double().T)
    if lo:          # (the activations between the two products are rounded to bfloat16: 2^-9 of their size)
        assert float((got.double() - want).abs().max()) <= 0.02 * float(want.abs().max())
        close = s.topk(min(top + 1, E), dim=1).values
        sure = (close[:, :-1] - close[:, 1:]).min(dim=1).values > 1e-4 if top < E else torch.ones(n, dtype=torch.bool)
        assert (sel.long()[sure] == s.topk(top, dim=1).indices[sure]).all()
    else:
        np.testing.assert_allclose(got.numpy(), want.numpy(), rtol=2e-4, atol=2e-5)
        assert (sel.long() == s.topk(top, dim=1).indices).all()           # best first
    # a token's rows do not depend on the batch around it: the same bits alone
    for t in (0, 7, n - 1):
        _, _, alone = run(h[t:t + 1])
        assert torch.equal(alone[0], rows_all[t])


def plain_recurrence_pieces(proj, w, width):
    """(u, output before the output projection) of the plain implementation for rows [branch | input]."""
    y = pb.gelu_tanh(proj[:, :width])
    u = pb.causal_conv(proj[:, width:], w["conv"], w["conv.b"])
    r, i = pb.block_gate(u, w["ra"], w["ra.b"]), pb.block_gate(u, w["ri"], w["ri.b"])
    log_a = -8.0 * r * pb.softplus(w["lam"])
    a = torch.exp(log_a)
    drive = torch.sqrt(1.0 - a * a) * i * u
    state, rows = torch.zeros_like(u[0]), []
    for t in range(u.shape[0]):
        state = a[t] * state + drive[t]
        rows.append(state)
    return u, torch.stack(rows) * y


@pytest.mark.parametrize("chunked", [False, True])
@pytest.mark.parametrize("width, blocks, taps", [(40, 2, 4), (48, 1, 1), (96, 3, 2), (130, 5, 7)])
def test_recurrence_carried_over_portions(width, blocks, taps, chunked):
    """Two requests in slots 3 and 1 of a dirty state array that is cleared for them, fed in portions of unequal
    sizes side by side (down to one token, shorter than the convolution); the result is that of each alone and whole."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(width)
    bw = width // blocks
    w = {"conv": 0.6 * torch.randn(width, taps, generator=g), "conv.b": 0.2 * torch.randn(width, generator=g),
         "ra": torch.randn(blocks, bw, bw, generator=g) / bw ** 0.5, "ra.b": 0.3 * torch.randn(blocks, bw, generator=g),
         "ri": torch.randn(blocks, bw, bw, generator=g) / bw ** 0.5, "ri.b": 0.3 * torch.randn(blocks, bw, generator=g),
         "lam": torch.empty(width).uniform_(-8.0, 1.0, generator=g)}
    lens = {3: 331, 1: 58}
    proj = {s: torch.randn(n, 2 * width, generator=g) for s, n in lens.items()}
    want = {s: plain_recurrence_pieces(proj[s].double(), {k: v.double() for k, v in w.items()}, width) for s in lens}
    state = torch.full((5, taps, width), 7.0, device="cuda")
    state[3].zero_(); state[1].zero_()
    gates = dev(torch.cat([w["ra"], w["ri"]], dim=1))
    cuts = {3: [1, 2, 64, 1, 3, 33, 27, 200], 1: [5, 1, 1, 2, 40, 9]}
    at = {s: 0 for s in lens}
    got_u = {s: [] for s in lens}
    got = {s: [] for s in lens}
    step = 0
    while any(at[s] < lens[s] for s in lens):
        live = [s for s in lens if at[s] < lens[s] and step < len(cuts[s])]
        parts = [proj[s][at[s]:at[s] + cuts[s][step]] for s in live]
        rows = dev(torch.cat(parts))
        counts = [p.shape[0] for p in parts]
        cu = dev(torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32))
        seq = dev(torch.tensor([i for i, c in enumerate(counts) for _ in range(c)], dtype=torch.int32))
        slots = dev(torch.tensor(live, dtype=torch.int32))
        u = ops.conv_step(rows, width, width, dev(w["conv"].t()), dev(w["conv.b"]), state, seq, cu, slots)
        assert ops.conv_step(rows, width, width, dev(w["conv"].t()), dev(w["conv.b"]), state, seq, cu, slots, rounded=True)[1].dtype == torch.bfloat16
        z = ops.head_product(u, gates, out_dtype=torch.float32)
        out = ops.rglru_scan(u, z, rows, branch_off=0, x_off=width, bias_r=dev(w["ra.b"].reshape(-1)), bias_i=dev(w["ri.b"].reshape(-1)),
                             lam=dev(w["lam"]), state=state, cu_tokens=cu, state_slots=slots, block_width=bw, decay=8.0, chunked=chunked)
        o = 0
        for s, c in zip(live, counts):
            got_u[s].append(u[o:o + c].cpu()); got[s].append(out[o:o + c].cpu())
            o += c; at[s] += c
        step += 1
    for s in lens:
        np.testing.assert_allclose(torch.cat(got_u[s]).numpy(), want[s][0].numpy(), rtol=1e-5, atol=1e-5)
        np.testing.assert_allclose(torch.cat(got[s]).numpy(), want[s][1].numpy(), rtol=2e-4, atol=2e-5)
    assert (state[[0, 2, 4]] == 7.0).all()                             # nobody else's row was touched


# ---- whole models under every cutting ---------------------------------------------------------------

@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, sharpen in CASES:
        cfg = CONFIGS[name]
        folder = write_model(str(tmp_path_factory.mktemp(f"buketar_{name}")), cfg, seed=11, sharpen=sharpen)
        _, tensors = pb.load_folder(folder)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(LENGTHS)}
        ref = {r: pb.forward(cfg, tensors, t).numpy().astype(np.float32) for r, t in reqs.items()}
        out[(name, sharpen)] = (folder, cfg, tensors, reqs, ref)
    return out


_ROUNDED = {}


def rounded_errors(key, models):
    """request -> the errors of the plain implementation in bfloat16 arithmetic, position by position."""
    if key not in _ROUNDED:
        folder, cfg, tensors, reqs, ref = models[key]
        some = {r: t for r, t in reqs.items() if len(t) <= 300}
        rounded = {r: pb.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in some.items()}
        _ROUNDED[key] = errors(rounded, ref, some)
    return _ROUNDED[key]


def errors(got, ref, reqs):
    scale = max(float(np.abs(v).max()) for v in ref.values())
    return {r: np.array([float(np.abs(got[r][p] - ref[r][p]).max()) / scale for p in range(len(t))]) for r, t in reqs.items()}


def worst(got, ref, reqs):
    scale = max(float(np.abs(v).max()) for v in ref.values())
    err, where = 0.0, None
    for r, toks in reqs.items():
        for p in range(len(toks)):
            e = float(np.abs(got[r][p] - ref[r][p]).max())
            if not e <= err:
                err, where = e, (r, p)
    return err / scale, where


def replay(folder, cfg, dtype, trace, out_dir, page=16, **kw):
    from inferrs_amd.engine import Engine, run_trace
    eng = Engine.from_folder(folder, dtype=dtype, page_size=page, num_pages=-(-trace.max_tokens // page), max_seqs=4, **kw)
    run_trace(eng, trace.lines, out_dir, io.StringIO())
    eng.cache.check_invariants()
    assert not eng.cache.sequences and all(g.pool.num_free == g.pool.num_pages for g in eng.cache.groups)
    assert eng.cache.slots.num_free == eng.cache.slots.num_slots
    return trace.read(out_dir, cfg["vocab"])


def traces(reqs):
    short = {r: t for r, t in reqs.items() if len(t) <= 65}
    return {
        "whole": tm.whole(reqs),
        "tail32": tm.prefix_then_single(reqs, 32),
        "every token alone": tm.prefix_then_single(short, 10 ** 6),
        "a long tail": tm.prefix_then_single({r: t for r, t in reqs.items() if 130 <= len(t) <= 300}, 120),
        "portions": tm.portions(reqs, [7, 2, 16, 3, 2, 33, 5, 2, 64]),
        "portions of two and three": tm.portions(short, [2, 3]),
        "mixed": tm.mixed(reqs, seed=1),
        "mixed2": tm.mixed(dict(reversed(list(reqs.items()))), seed=2, max_live=3),
    }


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0]}x{c[1]:g}")
def test_every_cutting_matches_plain(models, tmp_path, case, dtype):
    folder, cfg, tensors, reqs, ref = models[case]
    for mode, trace in traces(reqs).items():
        if mode.startswith("mixed"):
            assert trace.max_live >= 3 and trace.max_tokens < sum(tm.round_up(len(t), 64) for t in reqs.values())
        got = replay(folder, cfg, dtype, trace, str(tmp_path / f"{mode}_{dtype}"), page=16 if mode != "mixed2" else 32)
        part = {r: reqs[r] for r in got}
        if dtype == "float32":
            err, where = worst(got, ref, part)
            assert err <= TOL_F32, f"{case} {dtype} {mode}: {err:.3g} of the scale at {where}, allowed {TOL_F32:.3g}"
            continue
        plain = rounded_errors(case, models)
        common = [r for r in part if r in plain]
        mine = np.concatenate([errors(got, ref, part)[r] for r in common])
        theirs = np.concatenate([plain[r] for r in common])
        assert np.isfinite(np.concatenate(list(errors(got, ref, part).values()))).all(), f"{case} {mode}: not finite"
        for q, slack in ((0.5, 1.1), (0.9, 1.5)):
            a, b = float(np.quantile(mine, q)), float(np.quantile(theirs, q))
            assert a <= slack * b + 1e-3, f"{case} {dtype} {mode}: quantile {q} of the errors {a:.3g}, plain in bfloat16 {b:.3g}"


def test_sharpened_queries_see_far_keys(models):
    """What the sharpened models are for: taking the far half of the context away moves the logits by far more than
    any tolerance above, so the comparisons do rest on keys far back."""
    for case in [c for c in CASES if c[1] > 1.0]:
        folder, cfg, tensors, reqs, ref = models[case]
        toks = reqs["r8"]
        near = pb.forward(cfg, tensors, toks[350:]).numpy()
        scale = float(np.abs(ref["r8"]).max())
        moved = float(np.abs(near[-50:] - ref["r8"][-50:]).max()) / scale
        assert moved > 0.02, f"{case}: {moved}"


@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_scheduler(models, name):
    from inferrs_amd.engine import Engine
    from inferrs_amd.sampling import SamplingParams
    folder, cfg, tensors, reqs, ref = models[(name, 1.0)]
    prompts = [random_tokens(n, cfg["vocab"], 900 + n) for n in (1, 5, 40, 90, 17, 64)]
    n_new = [12, 30, 7, 20, 25, 3]
    eng = Engine.from_folder(folder, dtype="float32", page_size=8, num_pages=40, max_seqs=4)
    outs = eng.generate(prompts, [SamplingParams.greedy(max_tokens=n, bypass_stop_tokens=True) for n in n_new],
                        max_batch_size=3, max_tokens_per_step=48, prefill_chunk=16)
    for prompt, n, out in zip(prompts, n_new, outs):
        toks = list(prompt)
        for _ in range(n):
            toks.append(int(pb.forward(cfg, tensors, toks)[-1].argmax()))
        assert out.error is None and out.tokens == toks[len(prompt):]
    eng.cache.check_invariants()
    assert not eng.cache.sequences and eng.cache.slots.num_free == eng.cache.slots.num_slots


def test_random_weights_engine_steps():
    """The measurement script's way in: a configuration object and weights drawn on the device."""
    from inferrs_amd.config.buketar import BuketarConfig
    from inferrs_amd.engine import Engine
    from inferrs_amd.engine.engine import Entry
    eng = Engine.from_random(BuketarConfig.from_dict(CONFIGS["A"]), seed=1, dtype="bfloat16", page_size=16, num_pages=16, max_seqs=2)
    logits = eng.step([Entry("a", random_tokens(33, 211, 1), [32]), Entry("b", [5], [0])])
    assert logits.shape == (2, 211) and bool(torch.isfinite(logits).all())
    assert float(logits.abs().max()) <= 12.0


def test_trace_runner_program(models, tmp_path):
    folder, cfg, tensors, reqs, ref = models[("B", 1.0)]
    some = {r: reqs[r] for r in ("r2", "r3", "r4")}
    trace = tm.mixed(some, seed=5, max_live=2)
    out_dir = str(tmp_path / "out")
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", "float32", "--out", out_dir,
                        "--max-tokens", str(trace.max_tokens)], input=trace.text(), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(len(trace.lines))]
    err, where = worst(trace.read(out_dir, cfg["vocab"]), ref, some)
    assert err <= TOL_F32, (err, where)
