"""Milenex on the GPU: the HIP kernels against their fp32 references at odd, unaligned and
real-layer sizes in both element types; every mixer alone; planted keys; models served in float32
on every schedule within fp32 rounding of the oracle; bf16 models through HIP-graph decode and
eager mixed steps against the oracle and across schedules; graph vs eager; greedy generation."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import milenex_cases as mc  # noqa: E402
import milenex_oracle as mo  # noqa: E402
from ome_amd import ops  # noqa: E402
from ome_amd.ops import reference as ref  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF, F32 = torch.bfloat16, torch.float32
DTYPES = [F32, BF]
TOL, TYPICAL = 0.2, 0.03     # 16-bit whole-model runs: every position / the median of a request


def _close(got, want, dt, scale=1.0):
    err = (got.float().cpu() - want.float().cpu()).abs().max().item()
    assert err < (0.03 if dt == BF else 2e-5) * scale, err


# ------------------------------------------------------------------------------ kernels
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W", [7, 40, 192, 4096])
def test_shift_norm_kernel(dt, W):
    mc.shift_norm_case(DEV, dt, W=W)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,dim,vdim,K,rot,il", [(4, 2, 8, 6, 3, 4, True), (3, 3, 10, 4, 2, 10, True),
                                                      (4, 1, 70, 36, 5, 6, False), (1, 1, 8, 8, 0, 8, True),
                                                      (32, 8, 128, 128, 4, 64, True), (2, 1, 200, 256, 33, 0, True),
                                                      (6, 2, 96, 64, 1, 96, False), (4, 2, 16, 24, 3, 8, True),
                                                      (2, 2, 72, 40, 2, 72, True), (8, 2, 128, 128, 5, 64, True),
                                                      (2, 1, 256, 256, 6, 128, True), (3, 1, 64, 64, 1, 0, True)])
def test_conv_rope_cache_kernel(dt, Hq, Hkv, dim, vdim, K, rot, il):
    """Three sequences in one batch (a continued one, a fresh one on a dirty slot, a single row),
    two steps, against the reference op; caches and tails compared too."""
    g = torch.Generator().manual_seed(Hq * 100 + dim)
    from ome_amd.models.config import attn_tile_dim, plain_rope_table

    D, P, C = attn_tile_dim(max(dim, vdim)), 16, (Hq + Hkv) * dim + Hkv * vdim
    cs = plain_rope_table(100.0, rot, 256) if rot else torch.zeros(256, 0)
    wts = [(torch.randn(c, K, generator=g) * 0.5).to(dt) if K else None for c in (Hq * dim, Hkv * dim, Hkv * vdim)]
    state = {}
    for dev in ("cpu", DEV):
        tail = torch.full((5, max(K - 1, 0), C), 3.0, dtype=dt, device=dev) if K > 1 else None
        kc = torch.zeros(12, Hkv, P, D, dtype=dt, device=dev)
        vc = torch.zeros(12, Hkv, D, P, dtype=dt, device=dev)
        state[dev] = (tail, kc, vc, [])
    g2 = torch.Generator().manual_seed(5)
    base = [0, 0, 0]
    for step, lens in enumerate(([37, 1, 2], [3, 40, 1])):
        T = sum(lens)
        p = torch.randn(T, C + 3, generator=g2).to(dt)
        cu = torch.tensor([0, lens[0], lens[0] + lens[1], T], dtype=torch.int32)
        slot = torch.tensor([3, 1, 4], dtype=torch.int32)
        reset = torch.tensor([int(step == 0)] * 3, dtype=torch.int32)
        pos = torch.cat([torch.arange(base[s], base[s] + lens[s]) for s in range(3)]).to(torch.int32)
        slots = torch.cat([(s * 4 * P + torch.arange(base[s], base[s] + lens[s])) for s in range(3)]).to(torch.int32)
        slots[-1] = -1 if step == 1 else slots[-1]      # a padding row writes no cache entry
        for dev in ("cpu", DEV):
            tail, kc, vc, outs = state[dev]
            mv = lambda t: None if t is None else t.to(dev)   # noqa: E731
            pd = p.to(dev)
            q = torch.empty(T, Hq, D, dtype=dt, device=dev)
            ops.conv_rope_cache(pd[:, :Hq * dim], pd[:, Hq * dim:(Hq + Hkv) * dim], pd[:, (Hq + Hkv) * dim:C],
                                mv(wts[0]), mv(wts[1]), mv(wts[2]), tail, (cu.to(dev), slot.to(dev), reset.to(dev)),
                                pos.to(dev), cs.to(dev), rot, il, True, 1e-5, q, kc, vc, slots.to(dev), Hq, Hkv, dim, vdim)
            outs.append(q)
        base = [base[s] + lens[s] for s in range(3)]
    for a, b in zip(state["cpu"][3], state[DEV][3]):
        _close(b, a, dt)
    _close(state[DEV][1], state["cpu"][1], dt)
    _close(state[DEV][2], state["cpu"][2], dt, 4.0)
    if K > 1:
        assert torch.equal(state[DEV][0].cpu(), state["cpu"][0])


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,Hkv,D,vdim,window,ctx", [(6, 2, 64, 40, 9, 40), (4, 1, 64, 7, 6, 33), (1, 1, 64, 64, 0, 50),
                                                     (32, 8, 128, 128, 1024, 1500), (16, 1, 256, 200, 700, 900),
                                                     (18, 9, 64, 2, 20, 45), (32, 2, 128, 128, 0, 2100)])
def test_talking_attn_kernel(dt, H, Hkv, D, vdim, window, ctx):
    """Rows of three sequences at scattered pages and positions (first tokens, a window's edge, the
    longest context, a padding row), one chunk and several, against the reference op."""
    g = torch.Generator().manual_seed(H + ctx)
    P = 16
    n_pages = -(-ctx // P)
    kc = (torch.randn(3 * n_pages + 2, Hkv, P, D, generator=g) * 0.5).to(dt)
    vc = torch.randn(3 * n_pages + 2, Hkv, D, P, generator=g).to(dt)
    bt = torch.stack([torch.randperm(3 * n_pages, generator=g)[s * n_pages:(s + 1) * n_pages] + 1 for s in range(3)]).to(torch.int32)
    pos = torch.tensor([0, 1, ctx - 1, ctx - 2, max(window, 1) - 1, max(window, 1), ctx // 2, -1, 5, ctx - 1], dtype=torch.int32)
    pos = torch.where(pos >= ctx, torch.tensor(ctx - 1, dtype=torch.int32), pos)
    seq = torch.tensor([0, 1, 2, 0, 1, 2, 0, 0, 2, 1], dtype=torch.int32)
    T = pos.shape[0]
    q = (torch.randn(T, H, D, generator=g) * 0.5).to(dt)
    gate = torch.randn(T, H + 3, generator=g).to(dt)
    r1, r2 = torch.rand(H, generator=g), torch.rand(H, generator=g) * 2 + 0.1
    talk = torch.eye(H) + torch.randn(H, H, generator=g) * 0.3
    sinks = torch.randn(H, generator=g)
    want = ops.talking_attn(q, kc, vc, bt, seq, pos, 0.2, window, sinks, r1, r2, talk, gate[:, :H], vdim)
    d = lambda t: t.to(DEV)   # noqa: E731
    got = ops.talking_attn(d(q), d(kc), d(vc), d(bt), d(seq), d(pos), 0.2, window, d(sinks), d(r1), d(r2), d(talk),
                           d(gate)[:, :H], vdim)
    _close(got, want, dt, want.float().abs().max().item())
    got = ops.talking_attn(d(q), d(kc), d(vc), d(bt), d(seq), d(pos), 0.2, window, None, d(r1), d(r2), d(talk), None, vdim)
    want = ops.talking_attn(q, kc, vc, bt, seq, pos, 0.2, window, None, r1, r2, talk, None, vdim)
    _close(got, want, dt, want.float().abs().max().item())


@pytest.mark.parametrize("H,Hkv,D,vdim,window", [(6, 2, 64, 40, 9), (4, 1, 64, 7, 6), (32, 8, 128, 128, 100),
                                                 (16, 2, 256, 200, 0), (1, 1, 64, 64, 40), (18, 9, 64, 2, 20),
                                                 (12, 4, 128, 96, 33)])
def test_talking_prefill_kernel(H, Hkv, D, vdim, window):
    """Prompt chunks on the matrix-core kernel (fresh prompts, a chunk behind a prefix that crosses
    the window, a single row, row counts that do not fill a tile) against the row reference."""
    g = torch.Generator().manual_seed(H + D)
    P = 16
    q_lens, kv_lens = [37, 1, 50, 16], [37, 20, 150, 48]
    n_pages = [-(-k // P) for k in kv_lens]
    perm = (torch.randperm(sum(n_pages), generator=g) + 1).to(torch.int32)
    bt = torch.zeros(len(q_lens), max(n_pages), dtype=torch.int32)
    a = 0
    for s, n in enumerate(n_pages):
        bt[s, :n] = perm[a:a + n]
        a += n
    kc = (torch.randn(sum(n_pages) + 2, Hkv, P, D, generator=g) * 0.5).to(BF)
    vc = torch.randn(sum(n_pages) + 2, Hkv, D, P, generator=g).to(BF)
    T = sum(q_lens)
    q = (torch.randn(T, H, D, generator=g) * 0.5).to(BF)
    gate = torch.randn(T, H + 5, generator=g).to(BF)
    r1, r2 = torch.rand(H, generator=g), torch.rand(H, generator=g) * 2 + 0.1
    talk = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.3).to(BF).float()
    sinks = torch.randn(H, generator=g)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32)
    kl = torch.tensor(kv_lens, dtype=torch.int32)
    seq = torch.cat([torch.full((n,), s) for s, n in enumerate(q_lens)]).to(torch.int32)
    pos = torch.cat([torch.arange(k - n, k) for n, k in zip(q_lens, kv_lens)]).to(torch.int32)
    want = ops.talking_attn(q, kc, vc, bt, seq, pos, 0.2, window, sinks, r1, r2, talk, gate[:, :H], vdim)
    items = torch.tensor(ops.prefill_work_items(q_lens, kv_lens), dtype=torch.int32, device=DEV)
    d = lambda t: t.to(DEV)   # noqa: E731
    assert ops.talking_prefill_ok(d(q), H, D, P)
    got = ops.talking_prefill(d(q), d(kc), d(vc), d(bt), d(cu), d(kl), items, 0.2, window, d(sinks), d(r1), d(r2),
                              d(talk), d(gate)[:, :H], vdim)
    _close(got, want, BF, want.float().abs().max().item())
    got = ops.talking_prefill(d(q), d(kc), d(vc), d(bt), d(cu), d(kl), items, 0.2, window, None, d(r1), d(r2), d(talk),
                              None, vdim)
    want = ops.talking_attn(q, kc, vc, bt, seq, pos, 0.2, window, None, r1, r2, talk, None, vdim)
    _close(got, want, BF, want.float().abs().max().item())


@pytest.mark.parametrize("H,Hkv,D,vdim,window,ctx,B", [(6, 2, 64, 40, 150, 400, 4), (32, 8, 128, 128, 1024, 2100, 3),
                                                       (4, 1, 64, 7, 6, 33, 2), (16, 2, 256, 200, 0, 700, 5),
                                                       (12, 4, 128, 96, 0, 90, 70), (1, 1, 64, 64, 40, 50, 300)])
def test_talking_decode_kernel(H, Hkv, D, vdim, window, ctx, B):
    """Single rows with their keys split over workgroups (contexts of unequal length, one of a
    single token, a padding row of length 0) against the row reference."""
    g = torch.Generator().manual_seed(H + ctx)
    P = 16
    n_pages = -(-ctx // P)
    kc = (torch.randn(B * n_pages + 2, Hkv, P, D, generator=g) * 0.5).to(BF)
    vc = torch.randn(B * n_pages + 2, Hkv, D, P, generator=g).to(BF)
    bt = (torch.randperm(B * n_pages, generator=g) + 1).view(B, n_pages).to(torch.int32)
    lens = torch.randint(1, ctx + 1, (B,), generator=g).to(torch.int32)
    lens[0], lens[-1] = ctx, 1
    if B > 2:
        lens[1] = 0
    q = (torch.randn(B, H, D, generator=g) * 0.5).to(BF)
    gate = torch.randn(B, H + 5, generator=g).to(BF)
    r1, r2 = torch.rand(H, generator=g), torch.rand(H, generator=g) * 2 + 0.1
    talk = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.3).to(BF).float()
    sinks = torch.randn(H, generator=g)
    seq = torch.arange(B, dtype=torch.int32)
    want = ops.talking_attn(q, kc, vc, bt, seq, lens - 1, 0.2, window, sinks, r1, r2, talk, gate[:, :H], vdim)
    d = lambda t: t.to(DEV)   # noqa: E731
    got = ops.talking_decode(d(q), d(kc), d(vc), d(bt), d(lens), 0.2, window, d(sinks), d(r1), d(r2), d(talk),
                             d(gate)[:, :H], vdim)
    _close(got, want, BF, want.float().abs().max().item())


@pytest.mark.parametrize("dt", DTYPES)
def test_small_ops(dt):
    g = torch.Generator().manual_seed(2)
    for n in (40, 37, 4096 * 3):                         # GELU (erf), any length, both element types
        x = (torch.randn(n, generator=g) * 2).to(dt)
        _close(ops.act(x.to(DEV).clone(), 3), ref.act(x.clone(), 3), dt)
    for I in (24, 20, 4096):                             # clamped GLU with a per-row sigmoid gate
        x = (torch.randn(9, 2 * I, generator=g) * 2).to(dt)
        rg = torch.randn(9, 5, generator=g)
        got = ops.act_and_mul(x.to(DEV), 2, limit=0.75, row_gate=rg.to(DEV)[:, 3])
        _close(got, ref.act_and_mul(x, 2, 0.75, rg[:, 3]), dt)
    mc.route_excludes_groups_case(DEV)
    for E, k, ng, keep in ((16, 3, 2, 1), (12, 2, 3, 2), (64, 8, 8, 4), (5, 5, 1, 1)):
        logits = torch.randn(33, E + 1, generator=g)
        bias = torch.randn(E, generator=g) * 3 - 2
        a = ops.moe_route(logits[:, :E], k, False, "softmax", bias=bias, n_group=ng, topk_group=keep, group_mode=3 if ng > 1 else 0)
        b = ops.moe_route(logits.to(DEV)[:, :E], k, False, "softmax", bias=bias.to(DEV), n_group=ng, topk_group=keep,
                          group_mode=3 if ng > 1 else 0)
        assert torch.equal(a[1].sort(-1).values, b[1].cpu().sort(-1).values)
        assert (a[0].sort(-1).values - b[0].cpu().sort(-1).values).abs().max() < 1e-6


# ------------------------------------------------------------------------------ mixers alone
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=8, vdim=8, conv=0, rot_dims=8),
                                dict(heads=3, kv_heads=3, dim=10, vdim=4, window=1000, conv=1, rot_dims=0, scale=1.3),
                                dict(heads=4, kv_heads=1, dim=70, vdim=36, window=3, conv=5, rot_dims=6, base=5000.0),
                                dict(heads=8, kv_heads=2, dim=128, vdim=128, window=40, conv=4, rot_dims=64, scale=0.09)])
def test_rotary_attention_alone(kw, dt):
    mc.mixer_alone(DEV, dt, mo.rotary_layer(**kw), T=70)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=8, vdim=8, window=1000),
                                dict(heads=4, kv_heads=1, dim=5, vdim=7, window=6, scale=0.9),
                                dict(heads=2, kv_heads=2, dim=36, vdim=70, window=1),
                                dict(heads=8, kv_heads=2, dim=128, vdim=128, window=40, scale=0.09)])
def test_biased_attention_alone(kw, dt):
    mc.mixer_alone(DEV, dt, mo.biased_layer(**kw), T=70)


@pytest.mark.parametrize("dt", DTYPES)
def test_feed_forwards_alone(dt):
    mc.dense_case(DEV, dt)
    mc.dense_case(DEV, dt, width=64, ff=100)
    for f, width in ((mo.moe(6, 2, 12, 20, groups=3, keep=2), 24), (mo.moe(4, 1, 9, 0, groups=2, keep=1, limit=0.8), 24),
                     (mo.moe(2, 2, 8, 0), 24), (mo.moe(8, 3, 32, 32, groups=4, keep=2, shared_limit=0.3), 64),
                     (mo.moe(6, 2, 64, 0, groups=1, keep=1), 96)):
        grouped = mc.moe_case(DEV, dt, f, width)
        assert grouped == (dt == BF and width % 32 == 0 and f["expert"]["ff"] % 32 == 0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_window_edge(kind, dt):
    for cuts in ([60], [55] + [1] * 5, [16, 16, 16, 12], mc.portions(60, [2, 3, 7])):
        mc.planted_window_case(DEV, dt, kind, 8, True, cuts)
        mc.planted_window_case(DEV, dt, kind, 9, False, cuts)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_far_key_and_page_borders(kind, dt):
    for back in (300, 303, 304, 319):
        mc.planted_far_case(DEV, dt, kind, 432, back, [400] + [1] * 32)
    mc.planted_far_case(DEV, dt, kind, 432, 415, mc.portions(432, [64, 35, 2, 17]))


# ------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", mc.config_a()), ("b", mc.config_b()), ("c", mc.config_c()), ("h", mc.config_bf16())):
        w = mo.make_weights(cfg, seed=11)
        out[name] = (cfg, w, mo.write_model(str(tmp_path_factory.mktemp("mil_" + name)), cfg, w), {})
    return out


def _schedules(toks):
    return (mc.whole_schedule(toks), mc.decode_schedule(toks, 24), mc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
            mc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31]))


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_float32_schedules_match_oracle(models, name):
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", mc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=1e-4)))
    eng = mc.make_engine(path, DEV, "float32", max_tokens=192)
    for sched in _schedules(toks):
        mc.assert_matches_oracle(eng, cfg, w, toks, sched, 2e-4, cache)
    assert eng.runner.launch_stats["decode-graph"] > 0


def test_bfloat16_schedules_match_oracle(models):
    cfg, w, path, cache = models["h"]
    toks = dict(zip("pqrstu", mc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=0.02)))
    outs = []
    for sched in _schedules(toks):
        eng = mc.make_engine(path, DEV, "bfloat16", max_tokens=192)
        outs.append(mc.assert_matches_oracle(eng, cfg, w, toks, sched, TOL, cache, TYPICAL))
    for o in outs[1:]:          # the same tokens under another schedule: only summation orders differ
        errs = torch.cat([mc.logit_errors(o[rid], outs[0][rid].double()) for rid in toks])
        assert errs.max().item() < TOL and errs.median().item() < 0.02


def test_slots_and_pages_are_reused(models):
    cfg, w, path, cache = models["h"]
    ps = mc.prompts(cfg, w, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25, 16, 30], seed=5, min_margin=0.02)
    toks = {f"r{i}": t for i, t in enumerate(ps)}
    for dt, tol, typ in (("bfloat16", TOL, TYPICAL), ("float32", 2e-4, None)):
        eng = mc.make_engine(path, DEV, dt, max_tokens=160)
        mc.assert_matches_oracle(eng, cfg, w, toks, mc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), tol, cache, typ)
        assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_graph_and_eager_decode_agree(models):
    cfg, w, path, cache = models["h"]
    toks = {"x": mc.prompts(cfg, w, [100], seed=9, min_margin=0.02)[0]}
    outs = []
    for graphs in (True, False):
        eng = mc.make_engine(path, DEV, "bfloat16", max_tokens=128, graphs=graphs)
        outs.append(mc.assert_matches_oracle(eng, cfg, w, toks, mc.decode_schedule(toks, 80), TOL, cache, TYPICAL)["x"])
        assert eng.runner.launch_stats["decode-graph"] > 0 if graphs else not eng.runner.launch_stats["decode-graph"]
    errs = mc.logit_errors(outs[0], outs[1].double())
    assert errs.max().item() < TOL and errs.median().item() < 0.01


def test_greedy_generation(models):
    cfg, w, path, _ = models["h"]
    ps = mc.prompts(cfg, w, [5, 19, 1], seed=13)
    for dt, clear in (("bfloat16", 0.25), ("float32", 1e-3)):
        eng = mc.make_engine(path, DEV, dt, max_tokens=256)
        got = mc.greedy_engine(eng, ps, 12)
        for p, g in zip(ps, got):
            want, gap = mc.greedy_reference(cfg, w, p, 12)
            assert len(g) == 12
            if gap > clear:                 # only clear-cut argmaxes are pinned
                assert g == want
