"""Milenex on the CPU path (fp32 reference ops) against the slow oracle: every mechanism alone,
then whole models through the engine's replay entry -- whole prompts, prefill + token-by-token
decoding, portions down to two tokens, batches of unequal requests, reused state slots and pages,
planted keys at the window's edge, far back and at page borders -- and greedy generation through
the scheduler."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import milenex_cases as mc  # noqa: E402
import milenex_oracle as mo  # noqa: E402
from ome_amd.models.config import ModelConfig, layer_runs  # noqa: E402

DEV, DT = "cpu", torch.float32


def test_oracle_sanity():
    mc.sink_matters_case()
    mc.mixing_matters_case()


def test_layer_runs():
    assert layer_runs({"layers": [0] * 4}) == [(0, 0), (1, 0), (2, 0), (3, 0)]
    assert layer_runs({"layers": [0] * 4, "loop": {"start": 1, "stop": 3, "times": 2}}) == \
        [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (3, 0)]
    assert layer_runs({"layers": [0] * 2, "loop": {"start": 0, "stop": 2, "times": 1}}) == [(0, 0), (1, 0)]
    assert layer_runs(mc.config_a()) == mo.layer_runs(mc.config_a())
    cfg = ModelConfig.from_hf(mc.config_a())
    assert cfg.num_layers == 8 and cfg.architecture == "Milenex"      # 1 + 3 x 2 + 1 layer runs


def test_shift_norm():
    mc.shift_norm_case(DEV, DT)
    mc.shift_norm_case(DEV, DT, W=7, seed=9)


@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=8, vdim=8, conv=0, rot_dims=8),
                                dict(heads=3, kv_heads=3, dim=10, vdim=4, window=1000, conv=1, rot_dims=0, scale=1.3),
                                dict(heads=4, kv_heads=1, dim=70, vdim=36, window=3, conv=5, rot_dims=6, base=5000.0),
                                dict(heads=2, kv_heads=2, dim=6, vdim=12, window=1, conv=2, rot_dims=6)])
def test_rotary_attention_alone(kw):
    mc.mixer_alone(DEV, DT, mo.rotary_layer(**kw))


@pytest.mark.parametrize("kw", [dict(), dict(heads=1, kv_heads=1, dim=8, vdim=8, window=1000),
                                dict(heads=4, kv_heads=1, dim=5, vdim=7, window=6, scale=0.9),
                                dict(heads=2, kv_heads=2, dim=36, vdim=70, window=1),
                                dict(heads=18, kv_heads=9, dim=4, vdim=2, window=20)])
def test_biased_attention_alone(kw):
    mc.mixer_alone(DEV, DT, mo.biased_layer(**kw))


def test_feed_forwards_alone():
    mc.dense_case(DEV, DT)
    for f, width in ((mo.moe(6, 2, 12, 20, groups=3, keep=2), 24), (mo.moe(4, 1, 9, 0, groups=2, keep=1, limit=0.8), 24),
                     (mo.moe(2, 2, 8, 0), 24), (mo.moe(8, 3, 32, 32, groups=4, keep=2, shared_limit=0.3), 64)):
        assert not mc.moe_case(DEV, DT, f, width)
    mc.moe_case(DEV, DT, mo.moe(8, 2, 12, 6, groups=2, keep=1), 24, correction=[-5.0, -5.2, -5.4, -5.6, -9, -9, -9, -9])
    mc.route_excludes_groups_case(DEV)


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_window_edge(kind):
    for cuts in ([60], [55] + [1] * 5, [16, 16, 16, 12], mc.portions(60, [2, 3, 7])):
        mc.planted_window_case(DEV, DT, kind, 8, True, cuts)       # the last key inside the window
        mc.planted_window_case(DEV, DT, kind, 9, False, cuts)      # the first one outside


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_far_key_and_page_borders(kind):
    for back in (300, 303, 304, 319):                              # keys 131 / 128 / 127 / 112 of 432 rows
        mc.planted_far_case(DEV, DT, kind, 432, back, [400] + [1] * 32)
    mc.planted_far_case(DEV, DT, kind, 432, 415, mc.portions(432, [64, 35, 2, 17]))   # key 16, in portions


# ------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", mc.config_a()), ("b", mc.config_b()), ("c", mc.config_c())):
        w = mo.make_weights(cfg, seed=11)
        out[name] = (cfg, w, mo.write_model(str(tmp_path_factory.mktemp("mil_" + name)), cfg, w), {})
    return out


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_schedules_match_oracle(models, name):
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", mc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=1e-4)))
    eng = mc.make_engine(path, DEV, "float32", max_tokens=192)
    for sched in (mc.whole_schedule(toks), mc.decode_schedule(toks, 24),
                  mc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]), mc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31])):
        mc.assert_matches_oracle(eng, cfg, w, toks, sched, 2e-4, cache)


def test_slots_and_pages_are_reused(models):
    cfg, w, path, cache = models["a"]
    ps = mc.prompts(cfg, w, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25], seed=5, min_margin=1e-4)
    toks = {f"r{i}": t for i, t in enumerate(ps)}
    eng = mc.make_engine(path, DEV, "float32", max_tokens=160)
    mc.assert_matches_oracle(eng, cfg, w, toks, mc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), 2e-4, cache)
    assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_long_decoding(models):
    """Eighty tokens one by one: every window of the stack passes over decoded tokens only."""
    cfg, w, path, cache = models["a"]
    toks = {"x": mc.prompts(cfg, w, [100], seed=9, min_margin=1e-4)[0]}
    eng = mc.make_engine(path, DEV, "float32", max_tokens=128)
    mc.assert_matches_oracle(eng, cfg, w, toks, mc.decode_schedule(toks, 80), 2e-4, cache)


def test_greedy_generation(models):
    cfg, w, path, _ = models["a"]
    ps = mc.prompts(cfg, w, [5, 19, 1], seed=13)
    eng = mc.make_engine(path, DEV, "float32", max_tokens=256)
    got = mc.greedy_engine(eng, ps, 10)
    for p, g in zip(ps, got):
        want, gap = mc.greedy_reference(cfg, w, p, 10)
        assert len(g) == 10
        if gap > 1e-3:                 # only clear-cut argmaxes are pinned
            assert g == want


def test_incomplete_checkpoint_is_refused(models, tmp_path):
    cfg, w, _, _ = models["b"]
    path = mo.write_model(str(tmp_path / "m"), cfg, {k: v for k, v in w.items() if k != "l1.mix.talk"})
    with pytest.raises(ValueError, match="talk"):
        mc.make_engine(path, DEV, "float32")
