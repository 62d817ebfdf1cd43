"""Scenarios shared by the CPU (fp32 reference ops) and GPU (HIP kernels) Milenex tests: every
mechanism alone against the slow oracle of ``milenex_oracle``, small random models run through the
engine's replay entry under different schedules, planted keys at the window's edge, far back and
at page borders.  The schedule builders are the ones of ``zavilorn_cases`` (they know nothing of a
design).  Every function takes the device and element type, so the two test files only bind them."""
from __future__ import annotations

import math
import random

import torch

import milenex_oracle as mo
from ome_amd import ops
from ome_amd.models.common import PagedKVCache
from ome_amd.models.mixers import ConvRotaryAttention, GeluMLP, GroupRoutedMoE, TalkingHeadsAttention
from zavilorn_cases import (chunked_schedule, decode_schedule, greedy_engine, make_engine, mixed_schedule,  # noqa: F401
                            portions, replay, run_chunks, whole_schedule)

F64 = torch.float64
BF = torch.bfloat16


def tol_of(dt):
    return 0.04 if dt == BF else 1e-4


def rel(got, want):
    return ((got.detach().cpu().to(F64) - want).abs().max() / want.abs().max()).item()


def w64(w):
    return {k: v.to(F64) for k, v in w.items()}


# ------------------------------------------------------------------------------------ configs
def config_a():
    """Biased attention first, a looped span of two layers run three times, sizes that are all
    different from each other, grouped routing with one of three groups kept, one layer without a
    feed-forward, a final layer after the loop."""
    return mo.make_config([
        mo.biased_layer(mlp=mo.dense(40)),
        mo.rotary_layer(mlp=mo.moe(6, 2, 12, 20, groups=3, keep=2)),
        mo.biased_layer(heads=4, kv_heads=1, dim=5, vdim=7, window=6, scale=0.9, mlp=None),
        mo.rotary_layer(heads=3, kv_heads=3, dim=10, vdim=4, window=11, conv=2, rot_dims=10, base=33.0, scale=0.4,
                        mlp=mo.moe(4, 1, 9, 0, groups=2, keep=1, limit=0.8)),
    ], loop=(1, 3, 3))


def config_b():
    """Other sizes and the values the first config keeps apart made equal, 1 or absent: no loop,
    rotary attention first, no convolution on one layer and a single tap on another, no rotation on
    one, one head, kv heads = heads, dim = vdim, a window longer than every prompt, one group,
    every expert chosen, head widths beyond one 64-wide tile."""
    return mo.make_config([
        mo.rotary_layer(heads=1, kv_heads=1, dim=8, vdim=8, window=1000, conv=0, rot_dims=8, base=7.0, scale=1.0,
                        mlp=mo.moe(2, 2, 8, 0)),
        mo.biased_layer(heads=1, kv_heads=1, dim=8, vdim=8, window=1000, scale=1.0, mlp=mo.dense(17)),
        mo.rotary_layer(heads=4, kv_heads=2, dim=70, vdim=36, window=3, conv=1, rot_dims=0, scale=0.2,
                        mlp=mo.moe(3, 1, 16, 8, shared_limit=0.5)),
        mo.biased_layer(heads=2, kv_heads=2, dim=36, vdim=70, window=1, scale=0.3, mlp=None),
    ], width=40, vocab=37, eps=1e-6)


def config_c():
    """The whole stack is the loop (start 0, stop = all layers), run twice; five taps."""
    return mo.make_config([mo.rotary_layer(conv=5, mlp=mo.dense(16)), mo.biased_layer(mlp=mo.moe(4, 2, 8, 8, groups=2, keep=2))],
                          width=16, vocab=29, loop=(0, 2, 2))


def config_bf16():
    """For 16-bit runs: kernel-friendly widths (grouped expert GEMMs), few routed evaluations."""
    return mo.make_config([
        mo.biased_layer(heads=4, kv_heads=2, dim=16, vdim=32, window=40, scale=0.25, mlp=mo.dense(96)),
        mo.rotary_layer(heads=4, kv_heads=1, dim=32, vdim=32, window=24, conv=3, rot_dims=16, scale=0.18,
                        mlp=mo.moe(4, 1, 32, 32, groups=2, keep=1)),
        mo.biased_layer(heads=2, kv_heads=2, dim=32, vdim=16, window=17, scale=0.2, mlp=mo.dense(64)),
    ], width=64, vocab=53, loop=(1, 3, 2))


def prompts(cfg, weights, lengths, seed=1, min_margin=0.0, cache=None):
    """Random prompts whose routed evaluations all have a clear router margin (a smaller one is a
    coin toss between the oracle and a 16- or 32-bit run)."""
    g = random.Random(seed)
    out = []
    for n in lengths:
        for _ in range(200):
            t = [g.randrange(cfg["vocab"]) for _ in range(n)]
            if min_margin <= 0 or mo.router_margin(cfg, weights, t) > min_margin:
                break
        else:
            raise AssertionError("no prompt with the wanted router margin")
        out.append(t)
    return out


def logit_errors(got, want):
    """Per position: rms over the vocabulary of the centred difference / rms of the oracle's
    centred logits over the request."""
    got, want = got.detach().cpu().to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()


def assert_matches_oracle(eng, cfg, weights, toks, schedule, tol, cache, typical=None):
    got = replay(eng, toks, schedule)
    for rid, t in toks.items():
        key = tuple(t)
        if key not in cache:
            cache[key] = mo.forward(cfg, weights, t)
        e = logit_errors(got[rid], cache[key])
        assert e.max().item() < tol, f"request {rid} ({len(t)} tokens): position {int(e.argmax())} differs from " \
                                     f"the oracle by {e.max().item():.3g} (limit {tol})"
        if typical is not None and len(t) > 4:
            assert e.median().item() < typical, f"request {rid}: median error {e.median().item():.3g}"
    return got


def greedy_reference(cfg, weights, prompt, n):
    t, gap = list(prompt), float("inf")
    for _ in range(n):
        lg = mo.forward(cfg, weights, t)[-1]
        top = torch.topk(lg, 2).values
        gap = min(gap, float(top[0] - top[1]))
        t.append(int(lg.argmax()))
    return t[len(prompt):], gap


# ------------------------------------------------------------------------------------ one mechanism
def rotary_block(m, width, dev, dt, max_pos=1024, pages=80, eps=1e-5):
    rot = m.get("rot") or {}
    blk = ConvRotaryAttention(0, width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"],
                              m.get("conv", 0), rot.get("base", 1.0), rot.get("dims", 0), m["scale"], eps, max_pos, dev, dt)
    return blk, PagedKVCache(1, pages, m["kv_heads"], blk.D, 16, dt, dev)


def biased_block(m, width, dev, dt, pages=80):
    blk = TalkingHeadsAttention(0, width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"], m["scale"],
                                dev, dt)
    return blk, PagedKVCache(1, pages, m["kv_heads"], blk.D, 16, dt, dev)


def mixer_alone(dev, dt, layer, width=24, T=45, cut_sets=None, seed=3):
    """One mixer over one sequence, whole and in portions, against the oracle."""
    cfg = mo.make_config([layer], width=width)
    w = mo.sub(mo.make_weights(cfg, seed), "l0.mix.")
    m = layer["mixer"]
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(seed))
    hq = h.to(dt).to(F64)
    rotary = layer["type"] == "attention"
    want = mo.rotary_attention(hq, w64(w), m, 1e-5) if rotary else mo.biased_attention(hq, w64(w), m)
    for cuts in cut_sets or ([T], [T - 5] + [1] * 5, portions(T, [2, 3, 17, 16, 1, 6])):
        blk, kv = (rotary_block if rotary else biased_block)(m, width, dev, dt)
        blk.load(w)
        got = run_chunks(blk, h.to(device=dev, dtype=dt), cuts, kv)
        assert rel(got, want) < tol_of(dt), (cuts, rel(got, want))


def shift_norm_case(dev, dt, W=40, seed=5):
    """Stream update + offset norm + token shift over a batch of three sequences (one continuing
    from an earlier step, one starting on a slot that held another sequence, one of a single row),
    against the oracle's functions applied per sequence."""
    g = torch.Generator().manual_seed(seed)
    lens_a, lens_b = [5, 0, 3], [4, 6, 1]          # step 1 / step 2 rows per sequence (sequence 1 starts in step 2)
    w = (torch.randn(W, generator=g) * 0.1).to(dt)
    mu = torch.rand(W, generator=g).to(dt)
    state = torch.full((6, W), 7.0, dtype=torch.float32, device=dev)     # dirty slots
    slots = [4, 2, 1]
    seqs_x = [torch.randn(lens_a[s] + lens_b[s], W, generator=g) for s in range(3)]
    seqs_y = [torch.randn(lens_a[s] + lens_b[s], W, generator=g).to(dt) for s in range(3)]
    want = [mo.token_shift(mo.offset_norm(x.to(F64) + y.to(F64), w.to(F64), 1e-5), mu.to(F64))
            for x, y in zip(seqs_x, seqs_y)]
    for step, lens in enumerate((lens_a, lens_b)):
        off = [0, 0, 0] if step == 0 else lens_a
        live = [s for s in range(3) if lens[s] > 0]
        x = torch.cat([seqs_x[s][off[s]:off[s] + lens[s]] for s in live]).to(dev)
        y = torch.cat([seqs_y[s][off[s]:off[s] + lens[s]] for s in live]).to(dev)
        cu = torch.tensor([0] + list(torch.tensor([lens[s] for s in live]).cumsum(0)), dtype=torch.int32, device=dev)
        slot = torch.tensor([slots[s] for s in live], dtype=torch.int32, device=dev)
        reset = torch.tensor([int(off[s] == 0) for s in live], dtype=torch.int32, device=dev)
        xin = x.clone()
        v, out = ops.shift_norm(x, w.to(dev), 1e-5, y, 1.0, None, 1.0, 1.0, mu.to(dev), state, (cu, slot, reset), dt)
        assert torch.equal(x, xin), "the shifted form must not write its input stream"
        a = 0
        for s in live:
            n = lens[s]
            assert rel(out[a:a + n], want[s][off[s]:off[s] + n]) < (0.02 if dt == BF else 1e-5), (step, s)
            assert rel(v[a:a + n], (seqs_x[s].to(F64) + seqs_y[s].to(F64))[off[s]:off[s] + n]) < 1e-6
            a += n
    # without a shift: in place, two addends with factors, plain weights
    x = torch.randn(7, W, generator=g).to(dev)
    y1, y2 = torch.randn(7, W, generator=g).to(dt).to(dev), torch.randn(7, W, generator=g).to(dt).to(dev)
    v64 = x.cpu().to(F64) + 0.5 * y1.cpu().to(F64) - 2.0 * y2.cpu().to(F64)
    r, out = ops.shift_norm(x, w.to(dev), 1e-5, y1, 0.5, y2, -2.0, 0.0, out_dtype=dt)
    assert r.data_ptr() == x.data_ptr() and rel(r, v64) < 1e-6
    assert rel(out, mo.rms_unit(v64, 1e-5) * w.to(F64)) < (0.02 if dt == BF else 1e-5)


def dense_case(dev, dt, width=24, ff=40):
    cfg = mo.make_config([mo.biased_layer(mlp=mo.dense(ff))], width=width)
    w = mo.sub(mo.make_weights(cfg, 8), "l0.mlp.")
    h = torch.randn(9, width, generator=torch.Generator().manual_seed(6)) * 2
    blk = GeluMLP(width, ff, dev, dt)
    blk.load(w)
    assert rel(blk.forward(h.to(device=dev, dtype=dt)), mo.dense_ff(h.to(dt).to(F64), w64(w))) < tol_of(dt)


def moe_block(f, width, dev, dt):
    r, sh, g = f["router"], f.get("shared") or {}, f["router"].get("groups") or {}
    return GroupRoutedMoE(width, r["experts"], r["top"], f["expert"]["ff"], f["expert"]["limit"], g.get("count", 1),
                          g.get("keep", 1), sh.get("ff", 0), sh.get("limit", 0.0), dev, dt)


def moe_case(dev, dt, f, width, rows=13, correction=None):
    """The routed feed-forward alone, on inputs whose router decisions are clear of ties."""
    cfg = mo.make_config([mo.biased_layer(mlp=f)], width=width)
    w = mo.sub(mo.make_weights(cfg, 9), "l0.mlp.")
    if correction is not None:
        w["correction"] = torch.tensor(correction, dtype=torch.float32).to(w["correction"].dtype)
    r = f["router"]
    for seed in range(7, 400):
        h = torch.randn(rows, width, generator=torch.Generator().manual_seed(seed))
        hq = h.to(dt).to(F64)
        s, _ = mo.route(hq, w64(w), r)
        c = (s + w["correction"].to(F64)).sort(-1, descending=True).values
        # margins inside the allowed groups are what matters; a global margin is the stricter test
        if r["top"] == r["experts"] or float((c[:, :-1] - c[:, 1:]).min()) > (2e-3 if dt == BF else 1e-5):
            break
    else:
        raise AssertionError("no input with the wanted router margin")
    blk = moe_block(f, width, dev, dt)
    blk.load(w)
    hd = h.to(device=dev, dtype=dt)
    got = blk.forward(hd)
    assert rel(got, mo.moe_ff(hq, w64(w), f)) < tol_of(dt)
    return blk.grouped_ok(hd)


def route_excludes_groups_case(dev):
    """Corrections so negative that every choice score of the best group lies below zero: an
    excluded expert must still lose against them (it counts as minus infinity, not as 0)."""
    E, top = 8, 2
    logits = torch.tensor([[2.0, 1.5, 0.1, 0.0, 1.0, 0.9, 0.8, 0.7],
                           [0.0, 0.1, 0.2, 0.3, 3.0, 0.5, 0.6, 2.0]], device=dev)
    bias = torch.tensor([-5.0, -5.2, -5.4, -5.6, -9.0, -9.0, -9.0, -9.0], device=dev)
    w, ids = ops.moe_route(logits, top, False, "softmax", bias=bias, n_group=2, topk_group=1, group_mode=3)
    s = torch.softmax(logits.cpu().double(), -1)
    assert sorted(ids[0].tolist()) == [0, 1] and sorted(ids[1].tolist()) == [0, 1]
    for t in range(2):
        for j in range(top):
            assert abs(float(w[t, j]) - float(s[t, int(ids[t, j])])) < 1e-6
    # the 0-for-excluded variant picks excluded experts here (0 > every allowed choice score)
    _, ids0 = ops.moe_route(logits, top, False, "softmax", bias=bias, n_group=2, topk_group=1, group_mode=1)
    assert any(i >= 4 for i in ids0[0].tolist()) and any(i >= 4 for i in ids0[1].tolist())


# ------------------------------------------------------------------------------------ planted keys
def _planted(dev, dt, layer, w, h, i, cuts, other_window, pages=80, moved=0.08):
    m = layer["mixer"]
    rotary = layer["type"] == "attention"
    f = (lambda hh, mm: mo.rotary_attention(hh, w64(w), mm, 1e-5)) if rotary else \
        (lambda hh, mm: mo.biased_attention(hh, w64(w), mm))
    hq = h.to(dt).to(F64)
    want = f(hq, m)
    blk, kv = (rotary_block if rotary else biased_block)(m, h.shape[1], dev, dt, pages=pages)
    blk.load(w)
    got = run_chunks(blk, h.to(device=dev, dtype=dt), cuts, kv)
    r = ((got[i].cpu().to(F64) - want[i]).abs().max() / want[i].abs().max()).item()
    assert r < tol_of(dt), r
    # the planted key matters: with the edge one token further / nearer the oracle's answer moves
    other = f(hq, dict(m, mask={"size": other_window}))
    assert (other[i] - want[i]).abs().max() > moved * want[i].abs().max()


def planted_layer(kind, window):
    """A layer whose keys are made by the query weights, with a sharp scale and nothing rotated or
    convolved, so that a doubled copy of the query's input row owns the softmax whenever visible."""
    if kind == "attention":
        L = mo.rotary_layer(heads=2, kv_heads=2, dim=16, vdim=16, window=window, conv=0, rot_dims=0, scale=6.0)
    else:
        L = mo.biased_layer(heads=2, kv_heads=2, dim=16, vdim=16, window=window, scale=1.5)
    w = mo.sub(mo.make_weights(mo.make_config([L], width=24), 6), "l0.mix.")
    w["k"] = w["q"].clone()
    if kind != "attention":
        w["talk"] = torch.eye(2).to(w["talk"].dtype)
        w["r1"] = torch.full_like(w["r1"], 0.25)
    return L, w


def planted_window_case(dev, dt, kind, gap, seen, cuts, T=60, window=9):
    """The planted key sits ``gap`` tokens behind the last row (window 9: gap 8 is the last key
    inside, gap 9 the first outside)."""
    L, w = planted_layer(kind, window)
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(4))
    h[T - 1 - gap] = 2 * h[T - 1]
    _planted(dev, dt, L, w, h, T - 1, cuts, window - 1 if seen else window + 1)


def planted_far_case(dev, dt, kind, T, back, cuts, window=1000):
    """One key hundreds of tokens back among hundreds of others, inside a long window; the other
    window used for the cross-check ends just short of it."""
    L, w = planted_layer(kind, window)
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(11))
    h[T - 1 - back] = 2 * h[T - 1]
    _planted(dev, dt, L, w, h, T - 1, cuts, back, pages=2 * (T // 16) + 12)


def sink_matters_case():
    """Leaving the sink out of the denominator changes the first rows most (few keys beside it)."""
    for L, f in ((mo.rotary_layer(), lambda h, w, m: mo.rotary_attention(h, w, m, 1e-5)),
                 (mo.biased_layer(), mo.biased_attention)):
        w = w64(mo.sub(mo.make_weights(mo.make_config([L]), 3), "l0.mix."))
        h = torch.randn(6, 24, generator=torch.Generator().manual_seed(3)).to(F64)
        a, b = f(h, w, L["mixer"]), f(h, dict(w, sink=torch.full_like(w["sink"], -1e9)), L["mixer"])
        assert (a[0] - b[0]).abs().max() > 0.1 * b[0].abs().max()


def mixing_matters_case():
    """The cross-head mix moves the output by an amount of its own size when taken away."""
    L = mo.biased_layer()
    w = w64(mo.sub(mo.make_weights(mo.make_config([L]), 3), "l0.mix."))
    h = torch.randn(12, 24, generator=torch.Generator().manual_seed(3)).to(F64)
    a = mo.biased_attention(h, w, L["mixer"])
    b = mo.biased_attention(h, dict(w, talk=torch.eye(L["mixer"]["heads"], dtype=F64)), L["mixer"])
    assert (a - b).abs().max() > 0.05 * a.abs().max()
    assert math.isfinite(float(a.abs().max()))
