"""Scenarios shared by the CPU (fp32 reference ops) and GPU (HIP kernels) Nivasun tests: every
mechanism alone against the slow oracle of ``nivasun_oracle``, small random models run through the
engine's replay entry under different schedules, planted keys at the window's edge, far back and
at page borders.  The schedule builders are the ones of ``zavilorn_cases`` (they know nothing of a
design).  Every function takes the device and element type, so the two test files only bind them."""
from __future__ import annotations

import random

import torch

import nivasun_oracle as no
from ome_amd import ops
from ome_amd.models.common import PagedKVCache
from ome_amd.models.mixers import DifferentialAttention, GroupRoutedMoE, KeyValuedAttention, LatentAttention
from zavilorn_cases import (chunked_schedule, decode_schedule, greedy_engine, make_engine, mixed_schedule,  # noqa: F401
                            portions, replay, run_chunks, whole_schedule)

F64 = torch.float64
BF = torch.bfloat16
EPS = 1e-5


def tol_of(dt):
    return 0.04 if dt == BF else 1e-4


def rel(got, want):
    return ((got.detach().cpu().to(F64) - want).abs().max() / want.abs().max()).item()


def w64(w):
    return {k: v.to(F64) for k, v in w.items()}


# ------------------------------------------------------------------------------------ configs
def config_a():
    """All three mixers, sizes that all differ from each other, a looped span of two layers run
    three times, one layer without a feed-forward, a final layer after the loop."""
    return no.make_config([
        no.diff_layer(mlp=no.moe(5, 2, 12, 10)),
        no.keyed_layer(mlp=no.moe(6, 3, 9, 0)),
        no.latent_layer(mlp=None),
        no.diff_layer(heads=3, kv_heads=3, dim=10, vdim=4, window=11, rot_dims=10, base=33.0, scale=0.4, diff=0.6,
                      mlp=no.moe(4, 1, 7, 20)),
    ], loop=(1, 3, 3))


def config_b():
    """Other sizes, and what the first config keeps apart made equal, 1 or absent: no loop, no pair
    table, no logit cap, one tap, one head, kv heads = heads, dim = vdim, windows longer than every
    prompt or of one token, every expert chosen, no shared expert, nothing rotated on one layer and
    the whole head on another, head widths beyond one 64-wide tile, a latent wider than the heads."""
    cfg = no.make_config([
        no.keyed_layer(heads=1, kv_heads=1, dim=8, window=1000, rot_dims=8, base=7.0, scale=1.0, mlp=no.moe(2, 2, 8, 0)),
        no.latent_layer(heads=1, dim=8, vdim=8, kv_rank=8, q_rank=8, window=1000, scale=1.0, mlp=no.moe(3, 1, 16, 8)),
        no.diff_layer(heads=4, kv_heads=2, dim=70, vdim=36, window=3, rot_dims=0, scale=0.2, diff=0.0, mlp=None),
        no.keyed_layer(heads=2, kv_heads=2, dim=72, window=1, rot_dims=0, scale=0.3, mlp=no.moe(4, 4, 5, 3)),
        no.latent_layer(heads=5, dim=4, vdim=12, kv_rank=70, q_rank=3, window=2, scale=0.7, mlp=None),
    ], width=40, vocab=37, eps=1e-6, taps=1, emb_scale=1.0, softcap=0.0)
    del cfg["embedding"]["bigram"]
    return cfg


def config_c():
    """The whole stack is the loop (start 0, stop = all layers), run twice; five taps; a pair
    table of one bucket; a layer with more query heads per kv head than one attention launch takes."""
    return no.make_config([no.latent_layer(mlp=no.moe(4, 2, 8, 8)), no.diff_layer(heads=2, kv_heads=1, mlp=no.moe(3, 2, 6, 0)),
                           no.keyed_layer(heads=34, kv_heads=2, dim=4, window=12, rot_dims=2, mlp=None)],
                          width=16, vocab=29, loop=(0, 3, 2), taps=5, buckets=1, mul_prev=1, mul_cur=1)


def config_bf16():
    """For 16-bit runs: kernel-friendly widths (grouped expert GEMMs, the 16-byte-vector kernels,
    the latent kernel's row shapes), few routed evaluations."""
    return no.make_config([
        no.diff_layer(heads=4, kv_heads=2, dim=16, vdim=32, window=40, rot_dims=8, scale=0.25, diff=0.4, mlp=no.moe(4, 1, 32, 32)),
        no.keyed_layer(heads=4, kv_heads=1, dim=32, window=24, rot_dims=16, scale=0.18, mlp=no.moe(4, 2, 32, 0)),
        no.latent_layer(heads=4, dim=16, vdim=16, kv_rank=48, q_rank=24, window=17, scale=0.25, mlp=no.moe(2, 1, 64, 32)),
    ], width=64, vocab=53, loop=(1, 3, 2))


def prompts(cfg, weights, lengths, seed=1, min_margin=0.0):
    """Random prompts whose routed evaluations all have a clear router margin (a smaller one is a
    coin toss between the oracle and a 16- or 32-bit run)."""
    g = random.Random(seed)
    out = []
    for n in lengths:
        for _ in range(200):
            t = [g.randrange(cfg["vocab"]) for _ in range(n)]
            if min_margin <= 0 or no.router_margin(cfg, weights, t) > min_margin:
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
            cache[key] = no.forward(cfg, weights, t)
        e = logit_errors(got[rid], cache[key])
        assert e.max().item() < tol, f"request {rid} ({len(t)} tokens): position {int(e.argmax())} differs from " \
                                     f"the oracle by {e.max().item():.3g} (limit {tol})"
        if typical is not None and len(t) > 4:
            assert e.median().item() < typical, f"request {rid}: median error {e.median().item():.3g}"
    return got


def greedy_reference(cfg, weights, prompt, n):
    t, gap = list(prompt), float("inf")
    for _ in range(n):
        lg = no.forward(cfg, weights, t)[-1]
        top = torch.topk(lg, 2).values
        gap = min(gap, float(top[0] - top[1]))
        t.append(int(lg.argmax()))
    return t[len(prompt):], gap


# ------------------------------------------------------------------------------------ one mechanism
def block_of(layer, width, dev, dt, max_pos=1024, pages=80):
    """The framework's block of a layer entry, with a one-layer paged cache of its shape."""
    m, kind = layer["mixer"], layer["type"]
    rot = m.get("rot") or {}
    if kind == "attention":
        blk = KeyValuedAttention(0, width, m["heads"], m["kv_heads"], m["dim"], m["mask"]["size"], rot.get("base", 1.0),
                                 rot.get("dims", 0), m["scale"], max_pos, dev, dt)
        return blk, PagedKVCache(1, pages, m["kv_heads"], blk.D, 16, dt, dev)
    if kind == "attention_2":
        blk = DifferentialAttention(0, width, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["mask"]["size"],
                                    rot.get("base", 1.0), rot.get("dims", 0), m["scale"], m["diff"], EPS, max_pos, dev, dt)
        return blk, PagedKVCache(1, pages, 2 * m["kv_heads"], blk.D, 16, dt, dev)
    blk = LatentAttention(0, 0, width, m["heads"], m["dim"], 0, m["vdim"], m["kv_rank"], m["q_rank"], 1.0, None,
                          m["scale"], EPS, max_pos, dev, dt, None, window=m["mask"]["size"], sink=False, gated=True)
    return blk, PagedKVCache(1, pages, 1, blk.D, 16, dt, dev, v_dim=0 if blk.latent_cache else None)


def oracle_mixer(layer, h, w):
    m = layer["mixer"]
    if layer["type"] == "attention":
        return no.key_valued_attention(h, w, m)
    if layer["type"] == "attention_2":
        return no.differential_attention(h, w, m, EPS)
    return no.latent_attention(h, w, m, EPS)


def mixer_alone(dev, dt, layer, width=24, T=45, cut_sets=None, seed=3):
    """One mixer over one sequence, whole and in portions, against the oracle."""
    cfg = no.make_config([layer], width=width, eps=EPS)
    w = no.sub(no.make_weights(cfg, seed), "l0.mix.")
    h = torch.randn(T, width, generator=torch.Generator().manual_seed(seed))
    want = oracle_mixer(layer, h.to(dt).to(F64), w64(w))
    for cuts in cut_sets or ([T], [T - 5] + [1] * 5, portions(T, [2, 3, 17, 16, 1, 6])):
        blk, kv = block_of(layer, width, dev, dt)
        blk.load(w)
        got = run_chunks(blk, h.to(device=dev, dtype=dt), cuts, kv)
        assert rel(got, want) < tol_of(dt), (cuts, rel(got, want))


def _batches(lens_a, lens_b, dev):
    """Two steps over three sequences (rows per sequence and step; 0 = not in the step): per step
    (live sequences, row offsets, cu, reset)."""
    for step, lens in enumerate((lens_a, lens_b)):
        off = [0, 0, 0] if step == 0 else lens_a
        live = [s for s in range(3) if lens[s] > 0]
        cu = torch.tensor([0] + list(torch.tensor([lens[s] for s in live]).cumsum(0)), dtype=torch.int32, device=dev)
        reset = torch.tensor([int(off[s] == 0) for s in live], dtype=torch.int32, device=dev)
        yield live, off, lens, cu, reset


def pair_embedding_case(dev, dt, W=24, V=41, buckets=13, mul_prev=5, mul_cur=3, seed=2):
    """Scaled embedding + hashed pair row over a batch of three sequences (one continuing from an
    earlier step, one starting on a slot that held another sequence, one of a single row): the
    previous token crosses the step border through the slot's state; a start takes the extra row."""
    g = torch.Generator().manual_seed(seed)
    emb = {"scale": 2.5, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}
    w = {"embed": torch.randn(V, W, generator=g).to(dt), "bigram": torch.randn(buckets + 1, W, generator=g).to(dt)}
    lens_a, lens_b = [5, 0, 3], [4, 6, 1]
    toks = [torch.randint(0, V, (lens_a[s] + lens_b[s],), generator=g).tolist() for s in range(3)]
    want = [no.embed_tokens(t, w64(w), emb) for t in toks]
    state = torch.full((6,), 7, dtype=torch.int32, device=dev)          # dirty slots
    slots = [4, 2, 1]
    for live, off, lens, cu, reset in _batches(lens_a, lens_b, dev):
        ids = torch.tensor(sum((toks[s][off[s]:off[s] + lens[s]] for s in live), []), dtype=torch.int32, device=dev)
        slot = torch.tensor([slots[s] for s in live], dtype=torch.int32, device=dev)
        x = ops.pair_embedding_f32(ids, w["embed"].to(dev), emb["scale"], w["bigram"].to(dev), buckets, mul_prev, mul_cur,
                                   state, (cu, slot, reset))
        assert x.dtype == torch.float32
        a = 0
        for s in live:
            assert rel(x[a:a + lens[s]], want[s][off[s]:off[s] + lens[s]]) < 1e-6, (s, off[s])
            a += lens[s]
    assert [int(state[slots[s]]) for s in range(3)] == [t[-1] for t in toks]
    # the extra row matters: taking the hashed row of "previous token 0" instead moves the first row
    other = w64(w)["embed"][toks[0][0]] * emb["scale"] + w64(w)["bigram"][(toks[0][0] * mul_cur) % buckets]
    assert (other - want[0][0]).abs().max() > 0.1


def stream_case(dev, dt, W=40, taps=3, seed=5):
    """Stream update with two addends and a pass vector, single-gain norm, then the residual
    convolution of the normed rows, over the same three-sequence batch in two steps."""
    g = torch.Generator().manual_seed(seed)
    gain = (1.0 + 0.2 * torch.randn((), generator=g)).to(dt)
    bias = torch.randn(W, generator=g).to(dt)
    cw = (torch.randn(W, taps, generator=g) * 0.4).to(dt)
    lens_a, lens_b = [5, 0, 3], [4, 6, 1]
    n = [lens_a[s] + lens_b[s] for s in range(3)]
    xs = [torch.randn(k, W, generator=g) for k in n]
    y1 = [torch.randn(k, W, generator=g).to(dt) for k in n]
    y2 = [torch.randn(k, W, generator=g).to(dt) for k in n]
    v64 = [x.to(F64) + a.to(F64) + b.to(F64) + bias.to(F64) for x, a, b in zip(xs, y1, y2)]
    h64 = [no.rms_unit(v, EPS) * gain.to(F64) for v in v64]
    state = torch.full((6, W, max(taps - 1, 0)), 3.0, dtype=torch.float32, device=dev)
    slots = [4, 2, 1]
    got_h = [[] for _ in range(3)]
    got_c = [[] for _ in range(3)]
    for live, off, lens, cu, reset in _batches(lens_a, lens_b, dev):
        cat = lambda seqs: torch.cat([seqs[s][off[s]:off[s] + lens[s]] for s in live]).to(dev)   # noqa: E731
        x = cat(xs)
        slot = torch.tensor([slots[s] for s in live], dtype=torch.int32, device=dev)
        r, h = ops.shift_norm(x, gain.expand(W).contiguous().to(dev), EPS, cat(y1), 1.0, cat(y2), 1.0, out_dtype=dt,
                              bias=bias.to(dev))
        assert r.data_ptr() == x.data_ptr()
        hc = ops.conv_mix(h, cw.to(dev), state, cu, slot, reset, dt)
        a = 0
        for s in live:
            assert rel(r[a:a + lens[s]], v64[s][off[s]:off[s] + lens[s]]) < 1e-6
            got_h[s].append(h[a:a + lens[s]].cpu())
            got_c[s].append(hc[a:a + lens[s]].cpu())
            a += lens[s]
    for s in range(3):
        h = torch.cat(got_h[s])
        assert rel(h, h64[s]) < (0.02 if dt == BF else 1e-5), s
        hq = h.to(F64)        # the convolution reads the rounded rows
        assert rel(torch.cat(got_c[s]), hq + no.causal_conv(hq, cw.to(F64))) < (0.02 if dt == BF else 1e-5), s


def diff_head_norm_case(dev, dt, T=9, G=2, R=3, D=64, vdim=10, lam=0.7, scale=0.6, seed=4):
    a = torch.randn(T, 2 * G * R, D, generator=torch.Generator().manual_seed(seed)).to(dt)
    v = a.to(F64).view(T, G, 2, R, D)[..., :vdim]
    want = (no.rms_unit(v[:, :, 0] - lam * v[:, :, 1], EPS) * scale).reshape(T, G * R * vdim)
    got = ops.diff_head_norm(a.to(dev), lam, EPS, scale, R, vdim)
    assert got.shape == (T, G * R * vdim) and rel(got, want) < (0.02 if dt == BF else 1e-5)


def moe_block(f, width, dev, dt):
    r, sh = f["router"], f.get("shared") or {}
    return GroupRoutedMoE(width, r["experts"], r["top"], f["expert"]["ff"], 0.0, 1, 1, sh.get("ff", 0), 0.0, dev, dt,
                          act=0, renorm=True, router_bias=True, correction=False)


def moe_case(dev, dt, f, width, rows=13):
    """The routed feed-forward alone, on inputs whose router decisions are clear of ties."""
    cfg = no.make_config([no.keyed_layer(mlp=f)], width=width)
    w = no.sub(no.make_weights(cfg, 9), "l0.mlp.")
    r = f["router"]
    for seed in range(7, 400):
        h = torch.randn(rows, width, generator=torch.Generator().manual_seed(seed))
        hq = h.to(dt).to(F64)
        c = no.router_logits(hq, w64(w)).sort(-1, descending=True).values
        if r["top"] == r["experts"] or float((c[:, :-1] - c[:, 1:]).min()) > (2e-2 if dt == BF else 1e-4):
            break
    else:
        raise AssertionError("no input with the wanted router margin")
    blk = moe_block(f, width, dev, dt)
    blk.load(w)
    hd = h.to(device=dev, dtype=dt)
    got = blk.forward(hd)
    assert rel(got, no.moe_ff(hq, w64(w), f)) < tol_of(dt)
    return blk.grouped_ok(hd)


def router_bias_case(dev):
    """The router's bias is part of the logits: it changes the choice AND the weights, which are
    the softmax over the chosen logits alone."""
    logits = torch.tensor([[2.0, 1.5, 0.1, 0.0, 1.0], [0.0, 0.1, 0.2, 0.3, 3.0]], device=dev)
    bias = torch.tensor([-3.0, 0.0, 0.0, 2.5, 0.0], device=dev)
    w, ids = ops.moe_route(logits, 2, True, "softmax", logit_bias=bias)
    z = (logits + bias).cpu().double()
    for t in range(2):
        val, idx = z[t].topk(2)
        assert sorted(ids[t].tolist()) == sorted(idx.tolist())
        p = torch.softmax(val, -1)
        for j in range(2):
            assert abs(float(w[t, j]) - float(p[idx.tolist().index(int(ids[t, j]))])) < 1e-6
    _, ids0 = ops.moe_route(logits, 2, True, "softmax")
    assert sorted(ids0[0].tolist()) == [0, 1] and sorted(ids[0].tolist()) == [1, 3]


# ------------------------------------------------------------------------------------ planted keys
def _planted(dev, dt, layer, w, h, i, cuts, other_window, pages=80, moved=0.08):
    m = layer["mixer"]
    hq = h.to(dt).to(F64)
    want = oracle_mixer(layer, hq, w64(w))
    blk, kv = block_of(layer, h.shape[1], dev, dt, pages=pages)
    blk.load(w)
    got = run_chunks(blk, h.to(device=dev, dtype=dt), cuts, kv)
    r = ((got[i].cpu().to(F64) - want[i]).abs().max() / want[i].abs().max()).item()
    assert r < tol_of(dt), r
    # the planted key matters: with the edge one token further / nearer the oracle's answer moves
    other = oracle_mixer(dict(layer, mixer=dict(m, mask={"size": other_window})), hq, w64(w))
    assert (other[i] - want[i]).abs().max() > moved * want[i].abs().max()


def planted_layer(kind, window):
    """A layer whose keys are made by the query weights, with a sharp scale and nothing rotated, so
    that a copy of the query's input row owns the softmax whenever visible.  ``plant(h, j, i)``
    makes row j the planted key of row i.  The differential layer plants its first map only (its
    weightless head norm cancels what both maps share).  The latent layer norms its latent, so a scaled copy
    would only tie with the row itself and carry the same value: there the keys are the NEGATED
    queries and the planted row is the negated input row (the row itself scores lowest)."""
    if kind == "attention":
        L = no.keyed_layer(heads=2, kv_heads=2, dim=16, window=window, rot_dims=0, scale=6.0)
    elif kind == "attention_2":
        L = no.diff_layer(heads=2, kv_heads=2, dim=16, vdim=12, window=window, rot_dims=0, scale=6.0, diff=0.3)
    else:
        L = no.latent_layer(heads=2, dim=16, vdim=12, kv_rank=20, q_rank=20, window=window, scale=0.6)
    w = no.sub(no.make_weights(no.make_config([L], width=24), 6), "l0.mix.")
    if kind == "latent_attention":
        w["dkv"], w["dkv.norm"], w["uk"] = w["dq"].clone(), w["dq.norm"].clone(), -w["uq"].clone()

        def plant(h, j, i):
            h[j] = -h[i]
    else:
        if kind == "attention_2":   # the first map only: the head norm would cancel a factor common to both maps
            w["k"] = torch.cat([w["q"].view(2, 2, 16, -1)[:, :1], w["k"].view(2, 2, 16, -1)[:, 1:]], 1).reshape(64, -1)
        else:
            w["k"] = w["q"].clone()

        def plant(h, j, i):
            h[j] = 2 * h[i]
    return L, w, plant


def planted_window_case(dev, dt, kind, gap, seen, cuts, T=60, window=9):
    """The planted key sits ``gap`` tokens behind the last row (window 9: gap 8 is the last key
    inside, gap 9 the first outside)."""
    L, w, plant = planted_layer(kind, window)
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(4))
    plant(h, T - 1 - gap, T - 1)
    _planted(dev, dt, L, w, h, T - 1, cuts, window - 1 if seen else window + 1)


def planted_far_case(dev, dt, kind, T, back, cuts, window=1000):
    """One key hundreds of tokens back among hundreds of others, inside a long window; the other
    window used for the cross-check ends just short of it."""
    L, w, plant = planted_layer(kind, window)
    h = torch.randn(T, 24, generator=torch.Generator().manual_seed(11))
    plant(h, T - 1 - back, T - 1)
    _planted(dev, dt, L, w, h, T - 1, cuts, back, pages=2 * (T // 16) + 12)


def constants_matter_case():
    """Oracle sanity: the sink, the temperature, the difference weight, the output gate, the pass
    vector of the FIRST pass and the logit cap each move the result by an amount of their own size."""
    h = torch.randn(12, 24, generator=torch.Generator().manual_seed(3)).to(F64)
    L = no.keyed_layer()
    w = w64(no.sub(no.make_weights(no.make_config([L]), 3), "l0.mix."))
    a = no.key_valued_attention(h, w, L["mixer"])
    b = no.key_valued_attention(h, dict(w, sink=torch.full_like(w["sink"], -1e9)), L["mixer"])
    assert (a[0] - b[0]).abs().max() > 0.1 * b[0].abs().max()
    c = no.key_valued_attention(h, dict(w, temp=torch.ones_like(w["temp"])), L["mixer"])
    assert (a - c).abs().max() > 0.02 * a.abs().max()
    L = no.diff_layer()
    w = w64(no.sub(no.make_weights(no.make_config([L]), 3), "l0.mix."))
    a = no.differential_attention(h, w, L["mixer"], EPS)
    b = no.differential_attention(h, dict(w, lq1=w["lq1"] + 1.0), L["mixer"], EPS)
    assert (a - b).abs().max() > 0.05 * a.abs().max()
    cfg = no.make_config([no.keyed_layer(mlp=no.moe())], loop=(0, 1, 2))
    wt = no.make_weights(cfg, 2)
    t = [3, 9, 1, 30, 7]
    a = no.forward(cfg, wt, t)
    step = wt["loop.step"].clone()
    step[0] = 0
    assert (a - no.forward(cfg, dict(wt, **{"loop.step": step}), t)).abs().max() > 0.05
    assert (a - no.forward(dict(cfg, logit_softcap=2.0), wt, t)).abs().max() > 0.05
