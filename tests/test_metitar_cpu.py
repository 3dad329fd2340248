"""Metitar on the CPU path (fp32 reference ops) against the slow oracle: every mechanism alone,
then whole models through the engine's replay entry -- whole prompts, prefill + token-by-token
decoding, portions down to two tokens, batches of unequal requests, reused state slots and pages,
planted keys far back and at page borders -- and greedy generation through the scheduler."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import metitar_cases as mc  # noqa: E402
import metitar_oracle as mo  # noqa: E402
from ome_amd import ops  # noqa: E402
from ome_amd.models.config import ModelConfig, yarn_rope_table  # noqa: E402
from ome_amd.models.mixers import Hgrn2Mixer, InputScaledMoE, PolyNormMLP, TokenSideInput  # noqa: E402

DEV, DT, TOL = "cpu", torch.float32, 2e-4
F64 = torch.float64


def _rel(got, want):
    return ((got.to(F64) - want).abs().max() / want.abs().max()).item()


def _w64(w):
    return {k: v.to(F64) for k, v in w.items()}


def _one_layer(layer, width=24, seed=3, **kw):
    cfg = mo.make_config([layer], width=width, **kw)
    return cfg, mo.random_weights(cfg, seed)


@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=8, rot_dim=8, vdim=8, kv_rank=8, q_rank=8, scaling=None),
                                dict(heads=5, dim=4, rot_dim=2, vdim=9, kv_rank=70, q_rank=5, base=5000.0, scale=1.3),
                                dict(heads=18, dim=4, rot_dim=4, vdim=2, kv_rank=6, q_rank=4)])
def test_latent_attention_alone(kw):
    L = mo.attention_layer(**kw)
    cfg, wt = _one_layer(L)
    w, m = mo.sub(wt, "l0.mix."), L["mixer"]
    h = torch.randn(45, 24, generator=torch.Generator().manual_seed(3))
    want = mo.latent_attention(h.to(F64), _w64(w), m, 1e-5)
    for cuts in ([45], [40] + [1] * 5, [2, 3, 17, 16, 1, 6]):
        blk, kv = mc.attention_block(m, 24, DEV, DT)
        blk.load(w)
        assert _rel(mc.run_chunks(blk, h, cuts, kv), want) < 1e-4, cuts


@pytest.mark.parametrize("kw", [dict(), dict(heads=5, dim=4, rot_dim=2, vdim=9, kv_rank=70, q_rank=5, scale=0.5),
                                dict(heads=18, dim=4, rot_dim=4, vdim=2, kv_rank=6, q_rank=4)])
def test_latent_attention_key_rows_layout(kw):
    """16-bit models keep one row per token that carries its own values (padded to a latent kernel
    shape): the same mixer on that layout, through the reference of the latent kernel."""
    L = mo.attention_layer(**kw)
    _, wt = _one_layer(L)
    w, m = mo.sub(wt, "l0.mix."), L["mixer"]
    h = torch.randn(45, 24, generator=torch.Generator().manual_seed(3)).to(torch.bfloat16)
    want = mo.latent_attention(h.to(F64), _w64(w), m, 1e-5)
    for cuts in ([45], [40] + [1] * 5, [2, 3, 17, 16, 1, 6]):
        blk, kv = mc.attention_block(m, 24, DEV, torch.bfloat16)
        blk.load(w)
        assert blk.latent_cache and (blk.D, blk.DV) in ops.LATENT_SHAPES
        assert _rel(mc.run_chunks(blk, h, cuts, kv), want) < 0.05, cuts


def test_sink_matters():
    """Leaving the sink out of the denominator changes the first rows most (few keys beside it)."""
    L = mo.attention_layer()
    _, wt = _one_layer(L)
    w, m = _w64(mo.sub(wt, "l0.mix.")), L["mixer"]
    h = torch.randn(6, 24, generator=torch.Generator().manual_seed(3)).to(F64)
    with_sink = mo.latent_attention(h, w, m, 1e-5)
    without = mo.latent_attention(h, dict(w, sink=torch.full_like(w["sink"], -1e9)), m, 1e-5)
    assert (with_sink[0] - without[0]).abs().max() > 0.2 * without[0].abs().max()


def test_rotary_table():
    for rot in (mo.attention_layer()["mixer"]["rot"], {"base": 50.0, "dims": 6},
                {"base": 3000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}}):
        cos, sin = mo.rotary_angles(rot, list(range(70)))
        tab = yarn_rope_table(rot["base"], rot["dims"], 70, rot.get("scaling")).to(F64)
        assert (tab - torch.cat([cos, sin], -1)).abs().max() < 1e-6
    sc = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}    # the scaling changes the table
    assert (yarn_rope_table(3000.0, 16, 70, sc) - yarn_rope_table(3000.0, 16, 70, None)).abs().max() > 0.1


@pytest.mark.parametrize("n,i,j", [(300, 299, 3), (300, 299, 0), (65, 64, 15), (65, 64, 16), (65, 64, 63), (40, 33, 32)])
@pytest.mark.parametrize("mode", ["whole", "decode", "portions"])
def test_planted_key_is_seen(n, i, j, mode):
    cuts = {"whole": [n], "decode": [i] + [1] * (n - i), "portions": mc.portions(n, [2, 15, 1, 31, 16])}[mode]
    mc.planted_key_case(DEV, DT, 1e-4, n, i, j, cuts)


@pytest.mark.parametrize("cuts", [[40], [30, 10], [33, 2, 5]])
def test_future_key_is_not_seen(cuts):
    mc.planted_key_case(DEV, DT, 1e-4, 40, 33, 34, cuts, seen=False)


@pytest.mark.parametrize("m", [dict(heads=2, dim=6, vdim=10), dict(heads=1, dim=8, vdim=8), dict(heads=3, dim=20, vdim=3),
                               dict(heads=2, dim=3, vdim=70)])
def test_hgrn2_alone(m):
    L = mo.hgrn2_layer(**m)
    _, wt = _one_layer(L, seed=4)
    w = mo.sub(wt, "l0.mix.")
    h = torch.randn(37, 24, generator=torch.Generator().manual_seed(2))
    blk = Hgrn2Mixer(24, m["heads"], m["dim"], m["vdim"], 1e-5, DEV, DT)
    blk.load(w)
    want = mo.hgrn2(h.to(F64), _w64(w), m, 1e-5)
    for cuts in ([37], [1] * 37, [3, 2, 1, 9, 22]):
        assert _rel(mc.run_chunks(blk, h, cuts), want) < 1e-4, cuts


def test_hgrn2_lower_bound_and_state_matter():
    L = mo.hgrn2_layer()
    _, wt = _one_layer(L, seed=4)
    w, m = _w64(mo.sub(wt, "l0.mix.")), L["mixer"]
    h = torch.randn(30, 24, generator=torch.Generator().manual_seed(2)).to(F64)
    want = mo.hgrn2(h, w, m, 1e-5)
    assert _rel(mo.hgrn2(h, dict(w, lower=torch.zeros_like(w["lower"])), m, 1e-5), want) > 0.05
    assert _rel(mo.hgrn2(h[10:], w, m, 1e-5), want[10:]) > 0.05        # a state that forgot its past shows


@pytest.mark.parametrize("taps", [2, 3, 5])
def test_conv_mix_alone(taps):
    g = torch.Generator().manual_seed(5)
    x, w = torch.randn(29, 12, generator=g), torch.randn(12, taps, generator=g) * 0.5
    want = x.to(F64) + mo.causal_conv(x.to(F64), w.to(F64))
    for cuts in ([29], [1] * 29, [2, 1, 20, 6]):
        st = torch.randn(3, 12, taps - 1, generator=g)       # stale tails: a first portion must not read them
        outs, a = [], 0
        for n in cuts:
            i32 = dict(dtype=torch.int32)
            outs.append(ops.conv_mix(x[a:a + n].contiguous(), w, st, torch.tensor([0, n], **i32), torch.tensor([2], **i32),
                                     torch.tensor([int(a == 0)], **i32), torch.float32))
            a += n
        assert _rel(torch.cat(outs), want) < 1e-5, cuts


@pytest.mark.parametrize("ff", [40, 13])
def test_polynorm_mlp_alone(ff):
    _, wt = _one_layer(mo.hgrn2_layer(mlp=mo.dense(ff)), seed=8)
    w = mo.sub(wt, "l0.mlp.")
    h = torch.randn(9, 24, generator=torch.Generator().manual_seed(6)) * 3
    blk = PolyNormMLP(24, ff, 1e-5, DEV, DT)
    blk.load(w)
    assert _rel(blk.forward(h), mo.polynorm_ff(h.to(F64), _w64(w), 1e-5)) < 1e-5


@pytest.mark.parametrize("f", [mo.moe(5, 2, 12, 20), mo.moe(3, 1, 9, 0), mo.moe(4, 4, 8, 8), mo.moe(12, 3, 32, 0)])
def test_input_scaled_moe_alone(f):
    _, wt = _one_layer(mo.hgrn2_layer(mlp=f), seed=9)
    w = mo.sub(wt, "l0.mlp.")
    h = torch.randn(31, 24, generator=torch.Generator().manual_seed(7))
    blk = InputScaledMoE(24, f["router"]["experts"], f["router"]["top"], f["expert"]["ff"],
                         (f.get("shared") or {}).get("ff", 0), DEV, DT)
    blk.load(w)
    assert mo.router_margin(h.to(F64), _w64(w), f) > 1e-5
    want = mo.moe_ff(h.to(F64), _w64(w), f)
    assert _rel(blk.forward(h), want) < 1e-5
    # scaling the expert's output instead of its input is another function
    s = torch.sigmoid(h.to(F64) @ w["router"].to(F64).T)
    alt = torch.zeros_like(want)
    for t in range(31):
        for e in torch.topk(s[t], f["router"]["top"]).indices.tolist():
            alt[t] += s[t, e] * mo.swiglu(h[t].to(F64), _w64(w), f"e{e}.")
    if f.get("shared"):
        alt = alt + mo.swiglu(h.to(F64), _w64(w), "shared.")
    assert _rel(alt, want) > 0.05


def test_token_side_input_alone():
    cfg, wt = _one_layer(mo.hgrn2_layer(), seed=10, side=4)
    cfg["layers"] = cfg["layers"] * 3          # the table holds three layers' slices; take the middle one
    table = torch.randn(cfg["vocab"], 12, generator=torch.Generator().manual_seed(1)).to(torch.bfloat16)
    w = mo.sub(wt, "l0.side.")
    toks = [5, 0, 52, 17, 5]
    x = torch.randn(5, 24, generator=torch.Generator().manual_seed(2))
    blk = TokenSideInput(24, 4, 4, DEV, DT)
    blk.load(w)
    res = x.clone()
    y = blk.forward(x, torch.tensor(toks, dtype=torch.int32), table.float())
    ops.post_norm_add(res, y, blk.norm, None, 1e-5, 1)
    want = x.to(F64) + mo.side_input(x.to(F64), toks, table.to(F64), _w64(w), 1, 4, 1e-5)
    assert _rel(res, want) < 1e-5


def test_post_norm_add():
    g = torch.Generator().manual_seed(3)
    res, y, w, b = (torch.randn(*s, generator=g) for s in ((7, 20), (7, 20), (20,), (20,)))
    y = y * 3 + 1.5
    r = res.clone()
    out = ops.post_norm_add(r, y, w, b, 1e-5, 0, torch.float32)
    want = res.to(F64) + mo.layer_norm(y.to(F64), w.to(F64), b.to(F64), 1e-5)
    assert _rel(r, want) < 1e-6 and _rel(out, want) < 1e-6
    r = res.clone()
    assert ops.post_norm_add(r, y, w, None, 1e-5, 1) is None
    assert _rel(r, res.to(F64) + mo.rms_unit(y.to(F64), 1e-5) * w.to(F64)) < 1e-6


def test_config_reader():
    cfg = mc.config_b()
    c = ModelConfig.from_hf(cfg)
    assert c.architecture == "Metitar" and c.hidden_size == 40 and c.vocab_size == 37 and c.num_layers == 4
    assert c.head_dim == 128 and c.num_heads == 5 and c.num_kv_heads == 1     # widest latent + rotary key: 72 -> 128


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", mc.config_a()), ("b", mc.config_b()), ("c", mc.config_c())):
        w = mo.random_weights(cfg, seed=11)
        out[name] = (cfg, w, mo.save_model(tmp_path_factory.mktemp("met_" + name), cfg, w), {})
    return out


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_schedules_match_oracle(models, name):
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", mc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=1e-4, cache=cache)))
    for sched in (mc.whole_schedule(toks), mc.decode_schedule(toks, 24), mc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
                  mc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31])):
        eng = mc.make_engine(path, DEV, "float32", max_tokens=192)   # 12 pages: the six requests share them in turn
        mc.assert_matches_oracle(eng, cfg, w, toks, sched, TOL, cache)


def test_residual_stream_matches_oracle(models):
    cfg, w, path, _ = models["a"]
    p = mc.prompts(cfg, w, [19], seed=4, min_margin=1e-4)[0]
    eng = mc.make_engine(path, DEV, "float32", max_tokens=64)
    eng.runner.model.debug_residuals = got = []
    eng.replay_step([("x", p, [18])], ["x"])
    want: list = []
    mo.forward(cfg, w, p, residuals=want)
    assert len(got) == len(want) == len(cfg["layers"])
    for a, b in zip(got, want):
        assert _rel(a, b) < 1e-4


def test_slots_and_pages_are_reused(models):
    """Twelve requests through four state slots and a pool smaller than their sum: a stale conv
    tail, recurrent state or key left by a finished request would show in a later one."""
    cfg, w, path, cache = models["a"]
    ps = mc.prompts(cfg, w, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25, 16, 30], seed=5, min_margin=1e-4, cache=cache)
    toks = {f"r{i}": t for i, t in enumerate(ps)}
    eng = mc.make_engine(path, DEV, "float32", max_tokens=160)
    mc.assert_matches_oracle(eng, cfg, w, toks, mc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), TOL, cache)
    assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_long_decoding(models):
    cfg, w, path, cache = models["a"]
    toks = {"x": mc.prompts(cfg, w, [100], seed=9, min_margin=1e-4, cache=cache)[0]}
    eng = mc.make_engine(path, DEV, "float32", max_tokens=128)
    mc.assert_matches_oracle(eng, cfg, w, toks, mc.decode_schedule(toks, 95), TOL, cache)


@pytest.mark.parametrize("name", ["a", "b"])
def test_greedy_generation(models, name):
    cfg, w, path, _ = models[name]
    ps = mc.prompts(cfg, w, [5, 19, 1], seed=13)
    eng = mc.make_engine(path, DEV, "float32", max_tokens=256)
    got = mc.greedy_engine(eng, ps, 12)
    for p, g in zip(ps, got):
        want, gap = mc.greedy_reference(cfg, w, p, 12)
        if gap > 1e-3:                      # (a near tie may legitimately flip)
            assert g == want
        else:
            assert g[:1] == want[:1]
