"""Nivasun on the GPU: the HIP kernels against their fp32 references at odd, unaligned and
real-layer sizes in both element types; every mixer alone; planted keys; models served in float32
on every schedule within fp32 rounding of the oracle; bf16 models through HIP-graph decode and
eager mixed steps against the oracle and across schedules; graph vs eager; greedy generation."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import nivasun_cases as nc  # noqa: E402
import nivasun_oracle as no  # noqa: E402
from ome_amd import ops  # noqa: E402
from ome_amd.models.config import attn_tile_dim, plain_rope_table  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF, F32 = torch.bfloat16, torch.float32
DTYPES = [F32, BF]
KINDS = ["attention", "attention_2", "latent_attention"]
TOL, TYPICAL = 0.2, 0.03     # 16-bit whole-model runs: every position / the median of a request


def _close(got, want, dt, scale=1.0):
    err = (got.float().cpu() - want.float().cpu()).abs().max().item()
    assert err < (0.03 if dt == BF else 2e-5) * scale, err


# ------------------------------------------------------------------------------ kernels
@pytest.mark.parametrize("dt", DTYPES)
def test_pair_embedding_kernel(dt):
    nc.pair_embedding_case(DEV, dt)
    nc.pair_embedding_case(DEV, dt, W=7, V=300, buckets=1, mul_prev=1000003, mul_cur=999983, seed=8)
    nc.pair_embedding_case(DEV, dt, W=2048, V=5000, buckets=4099, mul_prev=36313, mul_cur=27191, seed=9)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("W,taps", [(40, 3), (7, 2), (24, 5), (16, 1), (192, 4), (4096, 3), (2050, 32)])
def test_stream_norm_and_convolution_kernels(dt, W, taps):
    nc.stream_case(DEV, dt, W=W, taps=taps)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T,G,R,D,vdim", [(9, 2, 3, 64, 10), (3, 1, 1, 128, 70), (40, 4, 4, 128, 128), (5, 1, 16, 256, 256),
                                         (1100, 2, 2, 64, 64), (2, 9, 2, 64, 2)])
def test_diff_head_norm_kernel(dt, T, G, R, D, vdim):
    nc.diff_head_norm_case(DEV, dt, T=T, G=G, R=R, D=D, vdim=vdim, lam=0.55, scale=0.7, seed=T + D)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,dim,vdim,rot,il,rep,qs", [(4, 2, 8, 8, 4, False, 1, True), (8, 4, 6, 10, 4, True, 2, False),
                                                           (3, 3, 10, 10, 10, False, 1, True), (8, 2, 70, 36, 6, True, 2, False),
                                                           (32, 8, 128, 128, 64, False, 1, True), (16, 8, 64, 128, 32, True, 2, False),
                                                           (4, 4, 72, 40, 0, True, 4, True), (2, 1, 256, 256, 128, False, 1, True),
                                                           (12, 4, 32, 64, 8, True, 2, True)])
def test_wide_norm_rope_cache_scale_and_shared_values(dt, Hq, Hkv, dim, vdim, rot, il, rep, qs):
    """The prep kernel with a per-head query factor and value heads shared by several key heads
    (a padding row included), scalar and 16-byte-vector paths, against the reference op."""
    g = torch.Generator().manual_seed(Hq * 100 + dim)
    D, P, T = attn_tile_dim(max(dim, vdim)), 16, 45
    nq, nk, nv = Hq * dim, Hkv * dim, (Hkv // rep) * vdim
    cs = plain_rope_table(100.0, rot, 256) if rot else torch.zeros(256, 0)
    p = torch.randn(T, nq + nk + nv + 8, generator=g).to(dt)
    scale = (0.5 + torch.rand(Hq, generator=g)) if qs else None
    pos = torch.arange(100, 100 + T, dtype=torch.int32)
    slots = (torch.randperm(12 * P, generator=g)[:T]).to(torch.int32)
    slots[7] = -1
    res = {}
    for dev in ("cpu", DEV):
        q = torch.empty(T, Hq, D, dtype=dt, device=dev)
        kc = torch.zeros(12, Hkv, P, D, dtype=dt, device=dev)
        vc = torch.zeros(12, Hkv, D, P, dtype=dt, device=dev)
        pd = p.to(dev)
        ops.wide_norm_rope_cache(pd[:, :nq], pd[:, nq:nq + nk], pd[:, nq + nk:nq + nk + nv], pos.to(dev), cs.to(dev), rot, il,
                                 None, None, 0.0, q, kc, vc, slots.to(dev), Hq, Hkv, dim, vdim,
                                 q_scale=None if scale is None else scale.to(dev), v_rep=rep)
        res[dev] = (q, kc, vc)
    for a, b in zip(res["cpu"], res[DEV]):
        _close(b, a, dt, 4.0)


@pytest.mark.parametrize("H,R,window,ctx,T", [(4, 48, 17, 90, 60), (16, 128, 72, 400, 33), (5, 70, 1, 40, 9), (40, 200, 150, 700, 3),
                                              (2, 64, 1000, 300, 120), (20, 512, 64, 260, 2)])
def test_latent_kernel_with_a_window(H, R, window, ctx, T):
    """The 16-head latent kernel restricted to the last ``window`` keys (rows of unequal context,
    one of a single key; few rows so that the keys are split over workgroups) against the reference."""
    g = torch.Generator().manual_seed(H + ctx)
    DK, DV = ops.latent_shape(R, 0)
    P = 16
    n_pages = -(-ctx // P)
    cache = torch.zeros(3 * n_pages + 2, 1, P, DK)
    cache[..., :R] = torch.randn(3 * n_pages + 2, 1, P, R, generator=g) * 0.5
    cache = cache.to(BF)
    bt = (torch.randperm(3 * n_pages, generator=g) + 1).view(3, n_pages).to(torch.int32)
    rows = torch.randint(0, 3, (T,), generator=g).to(torch.int32)
    lens = torch.randint(1, ctx + 1, (T,), generator=g).to(torch.int32)
    lens[0], lens[-1] = ctx, 1
    q = torch.zeros(T, H, DK)
    q[..., :R] = torch.randn(T, H, R, generator=g) * 0.5
    q = q.to(BF)
    c3 = cache.view(-1, P, DK)
    want = ops.latent_attn(q, c3, bt, rows, lens, 0.3, DV, window=window)
    d = lambda t: t.to(DEV)   # noqa: E731
    got = ops.latent_attn(d(q), d(c3), d(bt), d(rows), d(lens), 0.3, DV, ops.MLAWorkspace(DEV), window=window)
    _close(got, want, BF, want.float().abs().max().item())
    other = ops.latent_attn(q, c3, bt, rows, lens, 0.3, DV, window=window + 1)     # one key more is another answer
    if window < ctx:
        assert (other[0].float() - want[0].float()).abs().max() > 1e-3


def test_router_with_a_logit_bias():
    nc.router_bias_case(DEV)
    g = torch.Generator().manual_seed(2)
    for E, k in ((16, 3), (12, 2), (64, 8), (5, 5), (1, 1), (300, 16)):
        logits = torch.randn(33, E + 1, generator=g)
        bias = torch.randn(E, generator=g) * 2
        a = ops.moe_route(logits[:, :E], k, True, "softmax", logit_bias=bias)
        b = ops.moe_route(logits.to(DEV)[:, :E], k, True, "softmax", logit_bias=bias.to(DEV))
        assert torch.equal(a[1].sort(-1).values, b[1].cpu().sort(-1).values)
        assert (a[0].sort(-1).values - b[0].cpu().sort(-1).values).abs().max() < 1e-6


# ------------------------------------------------------------------------------ mixers alone
@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=8, rot_dims=8),
                                dict(heads=3, kv_heads=3, dim=10, window=1000, rot_dims=0, scale=1.3),
                                dict(heads=4, kv_heads=1, dim=70, window=3, rot_dims=6, base=5000.0),
                                dict(heads=8, kv_heads=2, dim=128, window=40, rot_dims=64, scale=0.09),
                                dict(heads=34, kv_heads=2, dim=8, window=20, rot_dims=4)])
def test_key_valued_attention_alone(kw, dt):
    nc.mixer_alone(DEV, dt, no.keyed_layer(**kw), T=70)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=8, vdim=8, window=1000, rot_dims=8, diff=0.0),
                                dict(heads=4, kv_heads=1, dim=5, vdim=7, window=6, rot_dims=2, scale=0.9, diff=0.8),
                                dict(heads=2, kv_heads=2, dim=36, vdim=70, window=1, rot_dims=0),
                                dict(heads=8, kv_heads=2, dim=64, vdim=128, window=40, rot_dims=32, scale=0.12),
                                dict(heads=17, kv_heads=1, dim=6, vdim=4, window=20)])
def test_differential_attention_alone(kw, dt):
    nc.mixer_alone(DEV, dt, no.diff_layer(**kw), T=70)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=8, vdim=8, kv_rank=8, q_rank=8, window=1000),
                                dict(heads=5, dim=4, vdim=12, kv_rank=70, q_rank=3, window=2, scale=0.7),
                                dict(heads=18, dim=6, vdim=4, kv_rank=16, q_rank=9, window=20),
                                dict(heads=8, dim=64, vdim=64, kv_rank=256, q_rank=96, window=40, scale=0.12)])
def test_latent_attention_alone(kw, dt):
    nc.mixer_alone(DEV, dt, no.latent_layer(**kw), T=70)


@pytest.mark.parametrize("dt", DTYPES)
def test_feed_forward_alone(dt):
    for f, width in ((no.moe(), 24), (no.moe(6, 3, 9, 0), 24), (no.moe(2, 2, 8, 0), 24), (no.moe(1, 1, 8, 5), 24),
                     (no.moe(8, 3, 32, 32), 64), (no.moe(6, 2, 64, 0), 96)):
        grouped = nc.moe_case(DEV, dt, f, width)
        assert grouped == (dt == BF and width % 32 == 0 and f["expert"]["ff"] % 32 == 0)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kind", KINDS)
def test_window_edge(kind, dt):
    for cuts in ([60], [55] + [1] * 5, [16, 16, 16, 12], nc.portions(60, [2, 3, 7])):
        nc.planted_window_case(DEV, dt, kind, 8, True, cuts)
        nc.planted_window_case(DEV, dt, kind, 9, False, cuts)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kind", KINDS)
def test_far_key_and_page_borders(kind, dt):
    for back in (300, 303, 304, 319):
        nc.planted_far_case(DEV, dt, kind, 432, back, [400] + [1] * 32)
    nc.planted_far_case(DEV, dt, kind, 432, 415, nc.portions(432, [64, 35, 2, 17]))


# ------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", nc.config_a()), ("b", nc.config_b()), ("c", nc.config_c()), ("h", nc.config_bf16())):
        w = no.make_weights(cfg, seed=11)
        out[name] = (cfg, w, no.write_model(str(tmp_path_factory.mktemp("niv_" + name)), cfg, w), {})
    return out


def _schedules(toks):
    return (nc.whole_schedule(toks), nc.decode_schedule(toks, 24), nc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
            nc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31]))


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_float32_schedules_match_oracle(models, name):
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", nc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=1e-4)))
    eng = nc.make_engine(path, DEV, "float32", max_tokens=192)
    for sched in _schedules(toks):
        nc.assert_matches_oracle(eng, cfg, w, toks, sched, 2e-4, cache)
    assert eng.runner.launch_stats["decode-graph"] > 0


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_bfloat16_odd_sizes_run_every_schedule(models, name):
    """Sizes no vector kernel takes, in 16 bits, on every schedule: the typical position against
    the oracle and against the whole-prompt run (single positions of a tiny random model may flip a
    router decision in 16 bits, so only medians are pinned here)."""
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrs", nc.prompts(cfg, w, [1, 2, 37, 50], min_margin=0.004)))
    outs = []
    for sched in _schedules(toks):
        eng = nc.make_engine(path, DEV, "bfloat16", max_tokens=192)
        outs.append(nc.assert_matches_oracle(eng, cfg, w, toks, sched, 1e9, cache, 0.1))
    for o in outs[1:]:
        errs = torch.cat([nc.logit_errors(o[rid], outs[0][rid].double()) for rid in toks])
        assert errs.median().item() < 0.05


def test_bfloat16_schedules_match_oracle(models):
    cfg, w, path, cache = models["h"]
    toks = dict(zip("pqrstu", nc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=0.02)))
    outs = []
    for sched in _schedules(toks):
        eng = nc.make_engine(path, DEV, "bfloat16", max_tokens=192)
        outs.append(nc.assert_matches_oracle(eng, cfg, w, toks, sched, TOL, cache, TYPICAL))
    for o in outs[1:]:          # the same tokens under another schedule: only summation orders differ
        errs = torch.cat([nc.logit_errors(o[rid], outs[0][rid].double()) for rid in toks])
        assert errs.max().item() < TOL and errs.median().item() < 0.02


def test_slots_and_pages_are_reused(models):
    cfg, w, path, cache = models["h"]
    ps = nc.prompts(cfg, w, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25, 16, 30], seed=5, min_margin=0.02)
    toks = {f"r{i}": t for i, t in enumerate(ps)}
    for dt, tol, typ in (("bfloat16", TOL, TYPICAL), ("float32", 2e-4, None)):
        eng = nc.make_engine(path, DEV, dt, max_tokens=160)
        nc.assert_matches_oracle(eng, cfg, w, toks, nc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), tol, cache, typ)
        assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_graph_and_eager_decode_agree(models):
    cfg, w, path, cache = models["h"]
    toks = {"x": nc.prompts(cfg, w, [100], seed=9, min_margin=0.02)[0]}
    outs = []
    for graphs in (True, False):
        eng = nc.make_engine(path, DEV, "bfloat16", max_tokens=128, graphs=graphs)
        outs.append(nc.assert_matches_oracle(eng, cfg, w, toks, nc.decode_schedule(toks, 80), TOL, cache, TYPICAL)["x"])
        assert eng.runner.launch_stats["decode-graph"] > 0 if graphs else not eng.runner.launch_stats["decode-graph"]
    errs = nc.logit_errors(outs[0], outs[1].double())
    assert errs.max().item() < TOL and errs.median().item() < 0.01


def test_greedy_generation(models):
    cfg, w, path, _ = models["h"]
    ps = nc.prompts(cfg, w, [5, 19, 1], seed=13)
    for dt, clear in (("bfloat16", 0.25), ("float32", 1e-3)):
        eng = nc.make_engine(path, DEV, dt, max_tokens=256)
        got = nc.greedy_engine(eng, ps, 12)
        for p, g in zip(ps, got):
            want, gap = nc.greedy_reference(cfg, w, p, 12)
            assert len(g) == 12
            if gap > clear:                 # only clear-cut argmaxes are pinned
                assert g == want
