"""Zavilorn on the CPU path (fp32 reference ops) against the slow oracle: every mechanism alone,
then whole models through the engine's replay entry -- whole prompts, prefill + token-by-token
decoding, portions down to two tokens, batches of unequal requests, reused state slots and pages,
keys at the edges of the window and of the kept first tokens -- and greedy generation through the
scheduler."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import zavilorn_cases as zc  # noqa: E402
import zavilorn_oracle as zo  # noqa: E402
from ome_amd.models.config import ModelConfig  # noqa: E402
from ome_amd.models.mixers import ClampedGLU, GatedDeltaMixer, Mamba2Mixer  # noqa: E402

DEV, DT, TOL = "cpu", torch.float32, 2e-4
F64 = torch.float64


_run_chunks = zc.run_chunks


def _rel(got, want):
    return ((got.to(F64) - want).abs().max() / want.abs().max()).item()


@pytest.mark.parametrize("m", [dict(heads=2, vdim=8, state=12, groups=1, conv=4, norm_groups=2),
                               dict(heads=4, vdim=4, state=6, groups=4, conv=2, norm_groups=1),
                               dict(heads=3, vdim=5, state=7, groups=3, conv=7, norm_groups=3)])
def test_mamba2_alone(m):
    cfg = zo.make_config([{"type": "mamba2", "mixer": m, "mlp": None}], width=24)
    w = zo.sub(zo.random_weights(cfg, 3), "l0.mix.")
    h = torch.randn(23, 24, generator=torch.Generator().manual_seed(1))
    blk = Mamba2Mixer(24, m["heads"], m["vdim"], m["state"], m["groups"], m["conv"], m["norm_groups"], 1e-5, DEV, DT)
    blk.load(w)
    want = zo.mamba2(h.to(F64), {k: v.to(F64) for k, v in w.items()}, m, 1e-5)
    for cuts in ([23], [1] * 23, [2, 5, 1, 1, 14]):
        assert _rel(_run_chunks(blk, h, cuts), want) < 1e-4, cuts


@pytest.mark.parametrize("m", [dict(heads=2, kv_heads=1, dim=12, vdim=20, conv=3),
                               dict(heads=3, kv_heads=3, dim=5, vdim=4, conv=2),
                               dict(heads=4, kv_heads=2, dim=64, vdim=8, conv=5)])
def test_gated_delta_alone(m):
    cfg = zo.make_config([zo.parallel_layer(r_heads=m["heads"], r_kv_heads=m["kv_heads"], r_dim=m["dim"],
                                            r_vdim=m["vdim"], r_conv=m["conv"])], width=24)
    w = zo.sub(zo.random_weights(cfg, 4), "l0.mix.right.")
    h = torch.randn(21, 24, generator=torch.Generator().manual_seed(2))
    blk = GatedDeltaMixer(24, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"], 1e-5, DEV, DT)
    blk.load(w)
    want = zo.gated_delta(h.to(F64), {k: v.to(F64) for k, v in w.items()}, m, 1e-5)
    for cuts in ([21], [1] * 21, [3, 2, 1, 15]):
        assert _rel(_run_chunks(blk, h, cuts), want) < 1e-4, cuts


def _attention_block(a, width):
    return zc.attention_block(a, width, DEV, DT)


@pytest.mark.parametrize("kw", [dict(), dict(heads=4, kv_heads=4, dim=8, vdim=8, window=4, keep_first=0, rot_dims=8),
                                dict(heads=4, kv_heads=2, dim=66, vdim=30, window=17, keep_first=5, rot_dims=2)])
def test_window_attention_alone(kw):
    L = zo.parallel_layer(**kw)
    a = L["mixer"]["left"]
    cfg = zo.make_config([L], width=24)
    w = zo.sub(zo.random_weights(cfg, 5), "l0.mix.left.")
    h = torch.randn(45, 24, generator=torch.Generator().manual_seed(3))
    want = zo.window_attention(h.to(F64), {k: v.to(F64) for k, v in w.items()}, a, 1e-5)
    for cuts in ([45], [40] + [1] * 5, [2, 3, 17, 16, 1, 6]):
        blk, kv = _attention_block(a, 24)
        blk.load(w)
        assert _rel(_run_chunks(blk, h, cuts, kv), want) < 1e-4, cuts


@pytest.mark.parametrize("gap,seen", [(8, True), (9, False)])
@pytest.mark.parametrize("cuts", [[60], [59, 1], [7, 2, 30, 21]])
def test_window_edge_shows(gap, seen, cuts):
    zc.planted_window_case(DEV, DT, 1e-4, gap, seen, cuts)


@pytest.mark.parametrize("j,seen", [(2, True), (3, False)])
@pytest.mark.parametrize("cuts", [[50], [49, 1], [2, 2, 46]])
def test_kept_first_edge_shows(j, seen, cuts):
    zc.planted_kept_case(DEV, DT, 1e-4, j, seen, cuts)


@pytest.mark.parametrize("ff,limit", [(40, 1.25), (13, 0.5)])
def test_clamped_glu_alone(ff, limit):
    cfg = zo.make_config([zo.mamba_layer(ff=ff, limit=limit)], width=24)
    w = zo.sub(zo.random_weights(cfg, 8), "l0.mlp.")
    h = torch.randn(9, 24, generator=torch.Generator().manual_seed(6)) * 3
    blk = ClampedGLU(24, ff, limit, DEV, DT)
    blk.load(w)
    want = zo.clamped_glu(h.to(F64), {k: v.to(F64) for k, v in w.items()}, {"limit": limit})
    assert _rel(blk.forward(h), want) < 1e-5
    g = h.to(F64) @ w["gate"].to(F64).T
    assert (g > limit).any() and (g < -limit).any()      # the clamp is exercised, on one side only for the gate


def test_config_reader():
    cfg = zc.config_b()
    c = ModelConfig.from_hf(cfg)
    assert c.architecture == "Zavilorn" and c.hidden_size == 40 and c.vocab_size == 37 and c.num_layers == 3
    assert c.head_dim == 128 and c.num_heads == 4 and c.num_kv_heads == 2 and c.tie_word_embeddings


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", zc.config_a()), ("b", zc.config_b())):
        w = zo.random_weights(cfg, seed=11)
        out[name] = (cfg, w, zo.save_model(tmp_path_factory.mktemp("zav_" + name), cfg, w), {})
    return out


@pytest.mark.parametrize("name", ["a", "b"])
def test_schedules_match_oracle(models, name):
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", zc.prompts(cfg, [1, 2, 37, 70, 16, 33])))
    for sched in (zc.whole_schedule(toks), zc.decode_schedule(toks, 24), zc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
                  zc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31])):
        eng = zc.make_engine(path, DEV, "float32", max_tokens=192)   # 12 pages: the six requests share them in turn
        zc.assert_matches_oracle(eng, cfg, w, toks, sched, TOL, cache)


def test_slots_and_pages_are_reused(models):
    """Twelve requests through four state slots and a pool smaller than their sum: a stale conv
    tail, recurrent state or key left by a finished request would show in a later one."""
    cfg, w, path, cache = models["a"]
    toks = {f"r{i}": t for i, t in enumerate(zc.prompts(cfg, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25, 16, 30], seed=5))}
    eng = zc.make_engine(path, DEV, "float32", max_tokens=160)
    zc.assert_matches_oracle(eng, cfg, w, toks, zc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), TOL, cache)
    assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_long_decoding(models):
    cfg, w, path, cache = models["a"]
    toks = {"x": zc.prompts(cfg, [100], seed=9)[0]}
    eng = zc.make_engine(path, DEV, "float32", max_tokens=128)
    zc.assert_matches_oracle(eng, cfg, w, toks, zc.decode_schedule(toks, 95), TOL, cache)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation(models, name):
    cfg, w, path, _ = models[name]
    ps = zc.prompts(cfg, [5, 19, 1], seed=13)
    eng = zc.make_engine(path, DEV, "float32", max_tokens=256)
    got = zc.greedy_engine(eng, ps, 12)
    for p, g in zip(ps, got):
        want, gap = zc.greedy_reference(cfg, w, p, 12)
        if gap > 1e-3:                      # (a near tie may legitimately flip)
            assert g == want
        else:
            assert g[:1] == want[:1]
