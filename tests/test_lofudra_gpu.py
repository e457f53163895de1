"""Lofudra on the GPU against the plain implementation (`plain_lofudra.py`, 64-bit).

Mechanisms alone, through the kernels' Python face and the parts: the step between sub-layers of a stream with norms
on both sides, the softmax with a sink in every attention kernel (plain and matrix cores, keys split and not, prompts
and single tokens, the fused decode kernel) with a key that stands out just inside a window's edge and a stronger one
just outside it, and the three mixers with a matrix state carried from portion to portion in slots of a dirty state
array.  Then whole models through the engine's step function under every way of cutting the work (whole prompts, a
prompt and then token by token, every token alone, portions down to two tokens, up to four live requests mixed in a
pool whose pages and state slots are used again), in both precisions, with ordinary weights and with sharpened
queries.  Decays are drawn so that some heads remember for hundreds of tokens: a state that is lost, not cleared or
carried to the wrong request shows.  Greedy generation runs through the engine's own entry point and scheduler.

Tolerances.  32-bit: 2e-5 of the largest logit against the 64-bit result, at every position; where the plain
implementation's own 32-bit arithmetic is further off than a third of that (a head's output that nearly cancels in
front of its norm), three times what it is off.  bfloat16: the measure is
the distribution of the positions' errors against that of the plain implementation in bfloat16 arithmetic (every
operation rounded) on the same positions: the engine keeps more in 32-bit than that, so its median and its ninth
decile must not be larger (a tenth and a half of slack)."""
import io
import math
import os
import subprocess
import sys
from types import SimpleNamespace

import numpy as np
import pytest
import torch

import plain_lofudra as pl
import trace_modes as tm
from lofudra_configs import CONFIGS, random_tokens, write_model

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LENGTHS = [1, 2, 3, 17, 64, 65, 130, 300, 700]
TOL_F32 = 2e-5
CASES = [("A", 1.0), ("B", 1.0), ("C", 1.0), ("D", 1.0), ("E", 1.0), ("A", 6.0), ("B", 8.0), ("D", 5.0)]


def dev(t, dtype=None):
    return t.to(device="cuda", dtype=dtype or t.dtype).contiguous()


# ---- the step between sub-layers ------------------------------------------------------------------

@pytest.mark.parametrize("W", [40, 33, 300, 5000])
@pytest.mark.parametrize("y_dtype", [torch.float32, torch.bfloat16])
def test_step_between_sublayers(W, y_dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(W)
    n = 19
    x = torch.randn(n, W, generator=g)
    y, y2, rows_in = (torch.randn(n, W, generator=g).to(y_dtype) for _ in range(3))
    post, pre, vec = 1.0 + 0.1 * torch.randn(W, generator=g), 1.0 + 0.1 * torch.randn(W, generator=g), torch.randn(W, generator=g)
    xs = dev(x)
    h = ops.sandwich_step(xs, y=dev(y), y_scale=0.6, y2=dev(y2), y2_scale=1.1, post_weight=dev(post), post_eps=1e-5,
                          enter_rows=dev(rows_in), enter_vector=dev(vec), pre_weight=dev(pre), eps=1e-6, h_dtype=torch.float32)
    new = x.double() + pl.rms_norm(0.6 * y.double() + 1.1 * y2.double(), post.double(), 1e-5) + rows_in.double() + vec.double()
    np.testing.assert_allclose(xs.cpu().numpy(), new.numpy(), rtol=1e-5, atol=1e-5)
    np.testing.assert_allclose(h.cpu().numpy(), pl.rms_norm(new, pre.double(), 1e-6).numpy(), rtol=1e-4, atol=1e-5)
    # a read alone leaves the stream as it is; so does the model's end, which adds what is pending for some rows only
    before = xs.clone()
    h = ops.sandwich_step(xs, pre_weight=dev(pre), eps=1e-6, h_dtype=y_dtype)
    np.testing.assert_allclose(h.float().cpu().numpy(), pl.rms_norm(new, pre.double(), 1e-6).numpy(), rtol=2e-2 if y_dtype == torch.bfloat16 else 1e-4, atol=1e-2 if y_dtype == torch.bfloat16 else 1e-5)
    rows = torch.tensor([5, 0, 18], dtype=torch.int32)
    tail = ops.sandwich_step(xs, y=dev(y), post_weight=dev(post), post_eps=1e-5, rows=dev(rows), pre_weight=dev(pre), eps=1e-6,
                             h_dtype=torch.float32)
    end = new + pl.rms_norm(y.double(), post.double(), 1e-5)
    np.testing.assert_allclose(tail.cpu().numpy(), pl.rms_norm(end[rows.long()], pre.double(), 1e-6).numpy(), rtol=1e-4, atol=1e-5)
    assert torch.equal(xs, before)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_exact_gelu(dtype):
    from inferrs_amd import ops
    z = torch.linspace(-6, 6, 1001).to(dtype)
    got = ops.activation(dev(z.clone()), ops.state.ACT_GELU).float().cpu()
    np.testing.assert_allclose(got.numpy(), pl.gelu_erf(z.double()).numpy(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=2e-3 if dtype == torch.bfloat16 else 1e-6)


# ---- the softmax with a sink, at a window's edge ------------------------------------------------------

def sink_reference(q, kc, vc, positions, token_seq, table, window, scale):
    """Request by request on dense copies of its keys and values: p_j = exp(s_j) / (1 + sum exp(s_j))."""
    n, nq, d = q.shape
    nkv, page = kc.shape[1], kc.shape[2]
    out = torch.zeros(n, nq, d, dtype=torch.float64)
    for s in token_seq.unique().tolist():
        rows = (token_seq == s).nonzero().flatten()
        pos = positions[rows].long()
        length = int(pos.max()) + 1
        pages = table[s, :-(-length // page)].long()
        k = kc[pages].double().permute(1, 0, 2, 3).reshape(nkv, -1, d)[:, :length].repeat_interleave(nq // nkv, 0)
        v = vc[pages].double().permute(1, 0, 3, 2).reshape(nkv, -1, d)[:, :length].repeat_interleave(nq // nkv, 0)
        sc = torch.einsum("thd,hjd->thj", q[rows].double(), k) * scale
        j = torch.arange(length)
        hidden = j[None, :] > pos[:, None]
        if window:
            hidden |= j[None, :] < (pos[:, None] - window + 1)
        e = torch.exp(sc).masked_fill(hidden[:, None, :], 0.0)
        out[rows] = torch.einsum("thj,hjd->thd", e / (1.0 + e.sum(-1, keepdim=True)), v)
    return out


def sink_case(dtype, nq, nkv, d, page, lens, q_lens, window, seed):
    """Cached requests in shuffled pages (what lies beyond a request's length is NaN).  For every request's last query,
    head 0: the key just inside the window's edge (or, without a window, the request's first key) points along the
    query, and the key one place further back, outside the window, does so twice as strongly."""
    g = torch.Generator().manual_seed(seed)
    max_pages = max(-(-l // page) for l in lens)
    total = sum(-(-l // page) for l in lens) + 3
    perm = torch.randperm(total, generator=g).tolist()
    table = torch.zeros(len(lens), max_pages, dtype=torch.int32)
    for s, l in enumerate(lens):
        for j in range(-(-l // page)):
            table[s, j] = perm.pop()
    kc = torch.randn(total, nkv, page, d, generator=g).to(dtype)
    vc = torch.randn(total, nkv, d, page, generator=g).to(dtype)
    positions = torch.tensor([p for l, ql in zip(lens, q_lens) for p in range(l - ql, l)], dtype=torch.int32)
    token_seq = torch.tensor([s for s, ql in enumerate(q_lens) for _ in range(ql)], dtype=torch.int32)
    q = torch.randn(len(positions), nq, d, generator=g).to(dtype)
    for s, l in enumerate(lens):
        last = q[token_seq == s][-1, 0].float()
        inside = max(l - window, 0) if window else 0
        kc[int(table[s, inside // page]), 0, inside % page] = (last * 3).to(dtype)
        if window and inside > 0:
            kc[int(table[s, (inside - 1) // page]), 0, (inside - 1) % page] = (last * 6).to(dtype)
        for j in range(l, -(-l // page) * page):
            kc[int(table[s, j // page]), :, j % page] = float("nan")
            vc[int(table[s, j // page]), :, :, j % page] = float("nan")
    return q, kc, vc, positions, token_seq, table


def assert_close(got, want, rel, what):
    err = float((got.double().cpu() - want).abs().max()) / max(float(want.abs().max()), 1e-9)
    assert err <= rel, f"{what}: {err:.3g} of the scale, allowed {rel:.3g}"


SINK_LENS = [([1, 70, 129, 200, 64], [1, 70, 2, 1, 17]), ([300, 17, 1000, 33], [1, 1, 1, 1]), ([257], [257]), ([700, 40], [300, 1])]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,page,window", [(4, 2, 16, 4, None), (5, 1, 48, 16, 40), (6, 3, 12, 8, 17), (2, 2, 64, 16, 1)])
@pytest.mark.parametrize("lens,q_lens", SINK_LENS)
def test_sink_plain_kernel(dtype, nq, nkv, d, page, window, lens, q_lens):
    from inferrs_amd import ops
    q, kc, vc, positions, token_seq, table = sink_case(dtype, nq, nkv, d, page, lens, q_lens, window, 5)
    scale = 0.9 / math.sqrt(d)
    want = sink_reference(q, kc, vc, positions, token_seq, table, window, scale)
    for split in (None, False):
        got = ops.attention_generic(dev(q), dev(kc), dev(vc), dev(positions), dev(token_seq), dev(table), window=window,
                                    scale=scale, max_kv_len=max(lens), split=split, sink=True)
        assert_close(got, want, 1e-5 if dtype == torch.float32 else 2 ** -7, f"plain kernel split={split}")
    if not window:
        return
    # the sink is what makes the difference (among the few keys of a window)
    plain = ops.attention_generic(dev(q), dev(kc), dev(vc), dev(positions), dev(token_seq), dev(table), window=window,
                                  scale=scale, max_kv_len=max(lens))
    assert float((plain.double().cpu() - want).abs().max()) > 0.005


@pytest.mark.parametrize("nq,nkv,d,page,window", [(4, 2, 16, 16, None), (5, 1, 48, 16, 40), (8, 1, 128, 16, None), (32, 8, 128, 16, 300),
                                                  (2, 2, 64, 32, 24), (3, 3, 80, 16, 100), (2, 2, 256, 64, 1)])
@pytest.mark.parametrize("lens,q_lens", SINK_LENS)
def test_sink_matrix_cores(nq, nkv, d, page, window, lens, q_lens):
    from inferrs_amd import ops
    q, kc, vc, positions, token_seq, table = sink_case(torch.bfloat16, nq, nkv, d, page, lens, q_lens, window, 7)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    scale = 0.9 / math.sqrt(d)
    want = sink_reference(q, kc, vc, positions, token_seq, table, window, scale)
    for splits in (None, 1, 2, 8):
        got = ops.attention_mfma(dev(q), dev(kc), dev(vc), dev(positions), dev(cu), dev(table), max_q_len=max(q_lens),
                                 max_kv_len=max(lens), window=window, scale=scale, splits=splits, sink=True)
        assert_close(got, want, 2 ** -7, f"matrix cores splits={splits}")


@pytest.mark.parametrize("nq,nkv,d,page,window", [(8, 2, 128, 16, None), (4, 1, 64, 16, 40), (2, 2, 64, 32, None), (16, 2, 64, 16, 500)])
def test_sink_fused_decode(nq, nkv, d, page, window):
    """The decode kernel that norms, rotates, writes the cache and attends, with its keys split every way it offers:
    the same as the separate kernels with a sink."""
    from inferrs_amd import ops
    lens = [300, 17, 1000, 33, 64]
    g = torch.Generator().manual_seed(d + nq)
    q, kc, vc, positions, token_seq, table = sink_case(torch.bfloat16, nq, nkv, d, page, lens, [1] * len(lens), window, 9)
    n = len(lens)
    qkv = torch.randn(n, (nq + 2 * nkv) * d, generator=g).bfloat16()
    qw, kw = 1.0 + 0.1 * torch.randn(d, generator=g), 1.0 + 0.1 * torch.randn(d, generator=g)
    inv = torch.tensor([10000.0 ** (-2.0 * i / d) for i in range(d // 2)], dtype=torch.float32)
    cos, sin = ops.rope_table(dev(positions), dev(inv))
    slots = torch.tensor([int(table[s, (l - 1) // page]) * page + (l - 1) % page for s, l in enumerate(lens)], dtype=torch.int32)
    cu = torch.arange(n + 1, dtype=torch.int32)
    scale = 0.8 / math.sqrt(d)
    k1, v1 = dev(kc), dev(vc)
    qn = ops.qk_rope_kv(dev(qkv), nq, nkv, d, q_norm_w=dev(qw), k_norm_w=dev(kw), eps=1e-6, add_one=False, cos=cos, sin=sin,
                        rot=d, interleaved=False, k_cache=k1, v_cache=v1, slots=dev(slots), page_size=page)
    want = sink_reference(qn.cpu(), k1.cpu(), v1.cpu(), positions, token_seq, table, window, scale)
    for splits in (None, 1, 4, 32):
        k2, v2 = dev(kc), dev(vc)
        got = ops.attention_decode_fused(dev(qkv), k2, v2, dev(positions), dev(cu), dev(table), nq=nq, nkv=nkv, d=d,
                                         slots=dev(slots), q_norm_w=dev(qw), k_norm_w=dev(kw), eps=1e-6, add_one=False,
                                         cos=cos, sin=sin, max_kv_len=max(lens), window=window, scale=scale, splits=splits,
                                         sink=True)
        assert_close(got, want, 2 ** -6, f"fused decode splits={splits}")


# ---- the mixers with a matrix state, carried from portion to portion ---------------------------------------

def _mixer_case(kind, g):
    from inferrs_amd.config import spec as sp
    W = 40
    def mat(o, i): return torch.randn(o, i, generator=g) / i ** 0.5
    if kind == "retention":
        H, d, dv = 3, 10, 12
        m = {"heads": H, "dim": d, "vdim": dv, "decay": [0.999, 0.5, 0.97]}
        w = {"q": mat(H * d, W), "k": mat(H * d, W), "v": mat(H * dv, W), "g": mat(H * dv, W), "o": mat(W, H * dv)}
        return sp.RetentionSpec(W, H, d, dv, tuple(m["decay"]), 1e-5), m, w, pl.retention
    if kind == "mlstm":
        H, d, dv = 2, 24, 9
        m = {"heads": H, "dim": d, "vdim": dv, "gate_cap": 6.0}
        w = {"q": mat(H * d, W), "k": mat(H * d, W), "v": mat(H * dv, W), "g": mat(H * dv, W), "o": mat(W, H * dv),
             "norm": 1.0 + 0.2 * torch.randn(H * dv, generator=g), "i": 3.0 * mat(H, W), "i.b": torch.randn(H, generator=g),
             "f": 3.0 * mat(H, W), "f.b": torch.tensor([2.0, 5.0])}
        return sp.MatrixMemorySpec(W, H, d, dv, 6.0, 1e-5), m, w, pl.mlstm
    H, dv, N, G, taps, parts = 4, 6, 20, 2, 4, 3
    m = {"heads": H, "vdim": dv, "state": N, "groups": G, "conv": taps, "norm_groups": parts}
    ch = H * dv + 2 * G * N
    w = {"in": mat(2 * H * dv + 2 * G * N + H, W), "conv": 0.6 * torch.randn(ch, taps, generator=g), "conv.b": 0.2 * torch.randn(ch, generator=g),
         "dt_bias": torch.tensor([-3.0, -1.0, 0.0, 1.0]), "A_log": torch.tensor([-6.0, -3.0, 0.0, 1.0]),
         "D": 1.0 + 0.3 * torch.randn(H, generator=g), "norm": 1.0 + 0.2 * torch.randn(H * dv, generator=g), "o": mat(W, H * dv)}
    return sp.StateSpaceSpec(W, H, dv, N, G, taps, parts, 1e-5), m, w, pl.mamba2


@pytest.mark.parametrize("kind", ["retention", "mlstm", "mamba2"])
def test_matrix_state_carried_over_portions(kind):
    """Two requests in slots 3 and 1 of a dirty state array that is cleared for them, fed in portions of unequal sizes
    side by side (down to one token, shorter than the convolution); the result is that of each alone and whole."""
    from inferrs_amd.cache.storage import LayerCache
    from inferrs_amd.parts.base import part_class
    g = torch.Generator().manual_seed(len(kind))
    spec, m, w, plain = _mixer_case(kind, g)
    cls = part_class("mixer", spec)
    assert {k: tuple(v.shape) for k, v in cls.tensors(spec).items()} == {k: tuple(v.shape) for k, v in w.items()}
    part = cls(spec, dict(w), torch.float32, "cuda")
    lens = {3: 331, 1: 58}
    h = {s: torch.randn(n, 40, generator=g) for s, n in lens.items()}
    want = {s: plain(h[s].double(), {"x." + k: v.double() for k, v in w.items()}, "x.", m, 1e-5) for s in lens}
    floats = cls.cache_need(spec).shape[0]
    state = torch.full((5, floats), 7.0, device="cuda")
    state[3].zero_(); state[1].zero_()
    cuts = {3: [1, 2, 64, 1, 3, 33, 27, 200], 1: [5, 1, 1, 2, 40, 9]}
    at = {s: 0 for s in lens}
    got = {s: [] for s in lens}
    step = 0
    while any(at[s] < lens[s] for s in lens):
        live = [s for s in lens if at[s] < lens[s] and step < len(cuts[s])]
        parts = [h[s][at[s]:at[s] + cuts[s][step]] for s in live]
        counts = [p.shape[0] for p in parts]
        ctx = SimpleNamespace(cu_tokens=dev(torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32)),
                              token_seq=dev(torch.tensor([i for i, c in enumerate(counts) for _ in range(c)], dtype=torch.int32)),
                              state_slots=dev(torch.tensor(live, dtype=torch.int32)), stream=None, partial_sums=False,
                              max_q_len=max(counts))
        out = part.forward(ctx, dev(torch.cat(parts)), LayerCache(0, state=state)).cpu()
        o = 0
        for s, c in zip(live, counts):
            got[s].append(out[o:o + c]); o += c; at[s] += c
        step += 1
    for s in lens:
        np.testing.assert_allclose(torch.cat(got[s]).numpy(), want[s].numpy(), rtol=3e-4, atol=3e-5)
    assert (state[[0, 2, 4]] == 7.0).all()                             # nobody else's row was touched


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("C,ld,off,taps", [(64, 160, 32, 4), (56, 83, 24, 3), (128, 196, 64, 1), (8, 16, 8, 7)])
def test_convolution_with_its_tail(C, ld, off, taps, dtype):
    """Two requests fed in portions (shorter than the taps too) from slots 2 and 0 of a dirty state array: channel by
    channel and, for bfloat16 rows whose sizes allow it, eight channels a thread."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(C + taps)
    lens = {2: 90, 0: 37}
    x = {s: torch.randn(n, ld, generator=g).to(dtype) for s, n in lens.items()}
    w, bias = (0.6 * torch.randn(C, taps, generator=g)).to(dtype), (0.2 * torch.randn(C, generator=g)).to(dtype)
    want = {s: pl.silu(pl.causal_conv(x[s][:, off:off + C].double(), w.double(), bias.double())) for s in lens}
    state = torch.full((3, 5 + (taps - 1) * C), 7.0, device="cuda")
    state[2].zero_(); state[0].zero_()
    cuts = {2: [1, 2, 1, 40, 3, 43], 0: [5, 1, 1, 30]}
    at, got, step = {s: 0 for s in lens}, {s: [] for s in lens}, 0
    while any(at[s] < lens[s] for s in lens):
        live = [s for s in lens if at[s] < lens[s] and step < len(cuts[s])]
        counts = [cuts[s][step] for s in live]
        rows = dev(torch.cat([x[s][at[s]:at[s] + c] for s, c in zip(live, counts)]))
        cu = dev(torch.tensor([0] + list(np.cumsum(counts)), dtype=torch.int32))
        seq = dev(torch.tensor([i for i, c in enumerate(counts) for _ in range(c)], dtype=torch.int32))
        out = ops.conv_act_step(rows, off, C, dev(w.t()), dev(bias), state, 5, seq, cu, dev(torch.tensor(live, dtype=torch.int32))).cpu()
        o = 0
        for s, c in zip(live, counts):
            got[s].append(out[o:o + c]); o += c; at[s] += c
        step += 1
    for s in lens:
        np.testing.assert_allclose(torch.cat(got[s]).double().numpy(), want[s].numpy(), rtol=1e-2 if dtype == torch.bfloat16 else 1e-5,
                                   atol=1e-2 if dtype == torch.bfloat16 else 1e-5)
    assert (state[1] == 7.0).all() and (state[:, :5].cpu() == torch.tensor([[0.0], [7.0], [0.0]])).all()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,qh,dim,vdim,normaliser", [(3, 3, 10, 12, False), (4, 2, 24, 9, True), (2, 1, 128, 64, True), (8, 8, 64, 128, False),
                                                      (2, 2, 256, 16, True), (1, 1, 512, 8, False), (2, 1, 132, 40, False)])
def test_scan_in_chunks_is_the_walk(H, qh, dim, vdim, normaliser, dtype):
    """Three requests of unequal lengths in one step, from states that are not zero: chunks of 16 and of 64 tokens side
    by side give what the walk token by token gives, outputs and final states, up to rounding; so do decays that are
    constants of the heads."""
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(H * dim)
    lens = [150, 1, 333]
    n = sum(lens)
    q = dev(torch.randn(n, qh * dim, generator=g), dtype)
    k = dev(torch.randn(n, qh * dim, generator=g), dtype)
    v = dev(torch.randn(n, H * vdim, generator=g), dtype)
    log_a = dev(-torch.rand(n, H, generator=g) * torch.tensor([0.001, 0.05, 0.5, 3.0] * 2)[:H])
    b = dev(torch.rand(n, H, generator=g))
    decay = dev(torch.tensor([0.999, 0.5, 0.97, 1.0, 0.0, 0.9, 0.99, 0.8][:H]))
    skip = dev(torch.randn(H, generator=g))
    cu = dev(torch.tensor([0, 150, 151, 484], dtype=torch.int32))
    slots = dev(torch.tensor([2, 0, 3], dtype=torch.int32))
    floats = H * (vdim + int(normaliser)) * dim
    start = torch.randn(5, floats + 7, generator=g)

    def run(chunk, **gates):
        state = dev(start.clone())
        out = ops.linear_scan(q=q, q_off=0, q_heads=qh, k=k, k_off=0, k_heads=qh, v=v, v_off=0, heads=H, dim=dim, vdim=vdim,
                              state=state, s_off=7, cu_tokens=cu, state_slots=slots, skip=skip, q_scale=0.7, k_scale=dim ** -0.5,
                              normaliser=normaliser, max_q_len=333, chunk=chunk, **gates)
        outs = out if normaliser else (out,)
        return [o.cpu().double() for o in outs] + [state.cpu().double()]

    for gates in (dict(log_a=log_a, b=b), dict(decay=decay)):
        walk = run(0, **gates)
        assert torch.equal(walk[-1][[1, 4]], start[[1, 4]].double()) and torch.equal(walk[-1][:, :7], start[:, :7].double())
        for chunk, matrix_cores in ((16, 1), (64, 1), (None, 1), (16, 0), (64, 0), (128, 1)):
            # (what a chunk's start contributes: on the matrix cores in true 32-bit, or on the vector units)
            ops.library().ia_linear_scan_tune(matrix_cores)
            try:
                results = run(chunk, **gates)
            finally:
                ops.library().ia_linear_scan_tune(1)
            for got, want in zip(results, walk):
                scale = float(want.abs().max())
                assert float((got - want).abs().max()) <= 2e-5 * scale, (chunk, matrix_cores, float((got - want).abs().max()) / scale)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gates_of_long_portions_are_the_walk(dtype):
    from inferrs_amd import ops
    g = torch.Generator().manual_seed(3)
    H, lens = 3, [700, 1, 40]
    n = sum(lens)
    proj = dev(4.0 * torch.randn(n, 2 * H + 5, generator=g), dtype)
    bi, bf = dev(torch.randn(H, generator=g)), dev(torch.tensor([1.0, 4.0, -2.0]))
    cu = dev(torch.tensor([0, 700, 701, 741], dtype=torch.int32))
    slots = dev(torch.tensor([1, 2, 0], dtype=torch.int32))
    start = torch.randn(3, H + 2, generator=g)
    results = []
    for longest in (1, 700):            # 1: the walk a (request, head); 700: a block's threads side by side
        state = dev(start.clone())
        outs = ops.exp_gates(proj, 2, 2 + H, bi, bf, 7.0, state, 2, cu, slots, max_q_len=longest)
        results.append([o.cpu().double() for o in outs] + [state.cpu().double()])
    for got, want in zip(results[1], results[0]):
        assert float((got - want).abs().max()) <= 2e-5 * max(float(want.abs().max()), 1.0)


# ---- whole models under every cutting ---------------------------------------------------------------

@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, sharpen in CASES:
        cfg = CONFIGS[name]
        folder = str(tmp_path_factory.mktemp(f"lofudra_{name}"))
        tensors = write_model(folder, cfg, seed=11, sharpen=sharpen)
        reqs = {f"r{i}": random_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate(LENGTHS)}
        ref64 = {r: pl.forward(cfg, tensors, t) for r, t in reqs.items()}
        ref = {r: v.numpy().astype(np.float32) for r, v in ref64.items()}
        scale = max(float(v.abs().max()) for v in ref64.values())
        # what rounding alone does at every position: the plain implementation in 32-bit against itself in 64-bit
        NOISE[(name, sharpen)] = {r: ((pl.forward(cfg, tensors, t, dtype=torch.float32).double() - ref64[r]).abs().max(1).values
                                      / scale).numpy() for r, t in reqs.items()}
        out[(name, sharpen)] = (folder, cfg, tensors, reqs, ref)
    return out


_ROUNDED = {}
NOISE = {}


def rounded_errors(key, models):
    """request -> the errors of the plain implementation in bfloat16 arithmetic, position by position."""
    if key not in _ROUNDED:
        folder, cfg, tensors, reqs, ref = models[key]
        some = {r: t for r, t in reqs.items() if len(t) <= 300}
        rounded = {r: pl.forward(cfg, tensors, t, dtype=torch.bfloat16).float().numpy() for r, t in some.items()}
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
            for r, e in errors(got, ref, part).items():
                allowed = np.maximum(TOL_F32, 3.0 * NOISE[case][r])
                assert (e <= allowed).all(), (f"{case} {dtype} {mode}: {float(e[np.argmax(e / allowed)]):.3g} of the scale at "
                                              f"({r}, {int(np.argmax(e / allowed))}), allowed {float(allowed[np.argmax(e / allowed)]):.3g}")
            continue
        plain = rounded_errors(case, models)
        common = [r for r in part if r in plain]
        mine = np.concatenate([errors(got, ref, part)[r] for r in common])
        theirs = np.concatenate([plain[r] for r in common])
        assert np.isfinite(np.concatenate(list(errors(got, ref, part).values()))).all(), f"{case} {mode}: not finite"
        for q, slack in ((0.5, 1.1), (0.9, 1.5)):
            a, b = float(np.quantile(mine, q)), float(np.quantile(theirs, q))
            assert a <= slack * b + 1e-3, f"{case} {dtype} {mode}: quantile {q} of the errors {a:.3g}, plain in bfloat16 {b:.3g}"


def test_the_models_rest_on_what_the_tests_are_for(models):
    """A window that is one place off, a sink that is left out and a state that is lost each move the logits by far
    more than any tolerance above."""
    import copy
    folder, cfg, tensors, reqs, ref = models[("A", 6.0)]
    toks = reqs["r7"]
    scale = float(np.abs(ref["r7"]).max())
    for delta in (-1, 1):
        other = copy.deepcopy(cfg)
        for L in other["layers"]:
            if L["type"] == "parallel":
                L["mixer"]["left"]["mask"]["size"] += delta
        moved = float(np.abs(pl.forward(other, tensors, toks).numpy() - ref["r7"]).max()) / scale
        assert moved > 100 * TOL_F32, f"a window of {delta:+d}: {moved}"
    # the far half of the context taken away (the recurrences' states)
    near = pl.forward(cfg, tensors, toks[150:]).numpy()
    assert float(np.abs(near[-50:] - ref["r7"][-50:]).max()) / scale > 100 * TOL_F32


@pytest.mark.parametrize("name", ["A", "C", "E"])
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
            toks.append(int(pl.forward(cfg, tensors, toks)[-1].argmax()))
        assert out.error is None and out.tokens == toks[len(prompt):]
    eng.cache.check_invariants()
    assert not eng.cache.sequences and eng.cache.slots.num_free == eng.cache.slots.num_slots


def test_random_weights_engine_steps():
    """The measurement script's way in: a configuration object and weights drawn on the device."""
    from inferrs_amd.config.lofudra import LofudraConfig
    from inferrs_amd.engine import Engine
    from inferrs_amd.engine.engine import Entry
    eng = Engine.from_random(LofudraConfig.from_dict(CONFIGS["A"]), seed=1, dtype="bfloat16", page_size=16, num_pages=16, max_seqs=2)
    logits = eng.step([Entry("a", random_tokens(33, 211, 1), [32]), Entry("b", [5], [0])])
    assert logits.shape == (2, 211) and bool(torch.isfinite(logits).all())


def test_command_line_run_and_bench(models):
    """The command line serves the design as it serves the others: greedy tokens are the plain implementation's, a drawn run
    and the timing command finish."""
    import json
    folder, cfg, tensors, reqs, ref = models[("A", 1.0)]
    prompt = random_tokens(9, cfg["vocab"], 3)
    toks = list(prompt)
    for _ in range(6):
        toks.append(int(pl.forward(cfg, tensors, toks)[-1].argmax()))
    exe = [sys.executable, os.path.join(ROOT, "bin", "inferrs-amd")]
    common = ["--block-size", "16", "--max-blocks", "32", "--max-batch-size", "2"]
    proc = subprocess.run(exe + ["run", folder, ",".join(map(str, prompt)), "--dtype", "f32", "--temperature", "0",
                                 "--repetition-penalty", "1.0", "--max-tokens", "6"] + common, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == toks[len(prompt):]
    proc = subprocess.run(exe + ["run", folder, ",".join(map(str, prompt)), "--dtype", "bf16", "--seed", "5", "--max-tokens", "12",
                                 "--ignore-eos"] + common, capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    drawn = [int(t) for t in proc.stdout.split()]
    assert len(drawn) == 12 and all(0 <= t < cfg["vocab"] for t in drawn)
    proc = subprocess.run(exe + ["bench", folder, "--dtype", "bf16", "--prompt-len", "40", "--max-tokens", "8", "--runs", "2"] + common,
                          capture_output=True, text=True, timeout=300)
    assert proc.returncode == 0, proc.stderr[-2000:]
    rec = json.loads(proc.stdout.strip().splitlines()[-1])
    assert rec["prefill_tok_s"] > 0 and rec["decode_tok_s"] > 0


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
