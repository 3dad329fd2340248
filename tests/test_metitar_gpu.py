"""Metitar on gfx950: the HIP kernels added for it against their fp32 references (odd sizes and
strided views included, bf16 and float instantiations), single mixers in portions, planted keys,
then whole models through the engine (HIP-graph decode, eager mixed steps) against the slow fp64
oracle under the same schedules as the CPU tests -- in bfloat16 and served in float32."""
import os
import sys
import tempfile

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import metitar_cases as mc  # noqa: E402
import metitar_oracle as mo  # noqa: E402
from ome_amd import ops  # noqa: E402
from ome_amd.models.mixers import Hgrn2Mixer, InputScaledMoE, PolyNormMLP  # noqa: E402
from ome_amd.ops import reference as ref  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF, F32, F64 = torch.bfloat16, torch.float32, torch.float64
TOL, TYPICAL = 0.25, 0.03     # bf16 against an fp64 oracle: every position / the median (see assert_matches_oracle)
DTYPES = [BF, F32]


def _tol(dt):
    return 1e-2 if dt == BF else 2e-5


def _close(got, want, tol):
    want = want.float()
    return (got.float().cpu() - want).abs().max().item() <= tol * max(1.0, want.abs().max().item())


def _rel(got, want):
    return ((got.cpu().to(F64) - want).abs().max() / want.abs().max()).item()


def _seqs(lens, slots, resets):
    cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32)
    return cu, torch.tensor(slots, dtype=torch.int32), torch.tensor(resets, dtype=torch.int32)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("T,H", [(1, 48), (37, 336), (5, 1030), (3, 4096), (2, 9000)])
@pytest.mark.parametrize("view", [True, False])     # False: contiguous, 16-byte aligned rows (the vector kernels)
def test_post_norm_add_and_row_norm(T, H, dt, view):
    torch.manual_seed(0)
    res, y = torch.randn(T, H) * 4, (torch.randn(T, H + 3) * 2 + 0.7).to(dt)[:, 3:]
    if not view:
        y = y.contiguous()
    w, b = (torch.rand(H) + 0.5).to(dt), (torch.randn(H) * 0.2).to(dt)
    for kind, bias in ((0, b), (1, None), (0, None)):
        r_ref = res.clone()
        want = ref.post_norm_add(r_ref, y, w, bias, 1e-6, kind, dt)
        r = res.to(DEV)
        got = ops.post_norm_add(r, y.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV), 1e-6, kind, dt)
        assert got.dtype == dt and _close(got, want, _tol(dt)) and _close(r, r_ref, 2e-5)
        r = res.to(DEV)
        assert ops.post_norm_add(r, y.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV), 1e-6, kind) is None
        assert _close(r, r_ref, 2e-5)
        assert _close(ops.row_norm(res.to(DEV), w.to(DEV), None if bias is None else bias.to(DEV), 1e-6, kind),
                      ref.row_norm(res, w, bias, 1e-6, kind), _tol(dt))
        assert _close(ops.row_norm(y.to(DEV), w.to(DEV), None, 1e-6, kind), ref.row_norm(y, w, None, 1e-6, kind), _tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("C,K,lens", [(328, 3, [1, 5, 130, 2]), (100, 7, [3, 70]), (64, 2, [1, 1, 1]), (24, 1, [9]),
                                      (300, 32, [200, 31, 33])])
def test_conv_mix(C, K, lens, dt):
    torch.manual_seed(1)
    S = len(lens)
    cu, slot, reset = _seqs(lens, [3, 1, 4, 2][:S], [1, 0, 1, 0][:S])
    T = int(cu[-1])
    x, w, st = torch.randn(T, C), (torch.randn(C, K) * 0.3).to(dt), torch.randn(6, C, K - 1)
    s_ref = st.clone()
    want = ref.conv_mix(x, w, s_ref, cu, slot, reset, torch.empty(T, C, dtype=dt))
    s = st.to(DEV)
    got = ops.conv_mix(x.to(DEV), w.to(DEV), s, cu.to(DEV), slot.to(DEV), reset.to(DEV), dt)
    assert _close(got, want, _tol(dt)) and torch.equal(s.cpu(), s_ref)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,d,vd,lens", [(5, 32, 64, [1, 9, 40]), (3, 48, 24, [17, 2]), (2, 128, 128, [20]),
                                         (5, 16, 64, [1, 1]), (2, 3, 70, [11]), (1, 128, 256, [9, 1]), (4, 64, 5, [30]), (1, 512, 64, [37]),
                                         (2, 128, 128, [300]), (40, 16, 64, [1] * 3)])
def test_hgrn2_scan(H, d, vd, lens, dt):
    torch.manual_seed(2)
    S = len(lens)
    cu, slot, reset = _seqs(lens, [2, 0, 3][:S], [0, 1, 0][:S])
    T = int(cu[-1])
    p = torch.randn(T, 2 * H * d + H * vd).to(dt)
    fb, lo, w, st = torch.randn(H * d).to(dt), torch.rand(H * d).to(dt), (torch.rand(vd) + 0.5).to(dt), torch.randn(4, H, d, vd)
    s_ref = st.clone()
    want = ref.hgrn2_scan(p[:, :H * d], p[:, H * d:2 * H * d], p[:, 2 * H * d:], fb, lo, w, s_ref, cu, slot, reset, H, d,
                          vd, 1e-6, torch.empty(T, H * vd, dtype=dt))
    pg, s = p.to(DEV), st.to(DEV)
    got = ops.hgrn2_scan(pg[:, :H * d], pg[:, H * d:2 * H * d], pg[:, 2 * H * d:], fb.to(DEV), lo.to(DEV), w.to(DEV), s,
                         cu.to(DEV), slot.to(DEV), reset.to(DEV), H, d, vd, 1e-6)
    assert _close(got, want, _tol(dt)) and _close(s, s_ref, 2e-5)


@pytest.mark.parametrize("dt", DTYPES)
def test_polynorm_gather_scale(dt):
    torch.manual_seed(3)
    coef = torch.tensor([0.9, -0.4, 0.3, 0.05])
    for T, F in ((5, 336), (70, 13), (3, 1030), (4, 14336), (2, 40000)):
        z = (torch.randn(T, F + 1) * 1.5).to(dt)[:, 1:]
        for zz in (z, z.contiguous()):      # a strided view, and aligned rows (the vector kernel)
            assert _close(ops.polynorm(zz.to(DEV), coef.to(DEV), 1e-6),
                          ref.polynorm(zz, coef, 1e-6, torch.empty(T, F, dtype=dt)), _tol(dt))
    g, ids, tab = torch.randn(9, 12).to(dt), torch.randint(0, 50, (9,), dtype=torch.int32), torch.randn(50, 60).to(dt)
    assert _close(ops.gelu_gather_mul(g.to(DEV), ids.to(DEV), tab.to(DEV), 24),
                  ref.gelu_gather_mul(g, ids, tab, 24, torch.empty_like(g)), _tol(dt))
    x, tw = torch.randn(7, 330).to(dt), torch.rand(7, 3)
    assert _close(ops.scale_rows(x.to(DEV), tw.to(DEV)), ops.scale_rows(x, tw), _tol(dt))


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("H,qlr,lat,rope,nope,D,off,own,vals", [
    (4, 80, 72, 32, 24, 128, 72, True, True), (3, 10, 12, 4, 8, 64, 12, True, True),
    (5, 7, 200, 56, 6, 256, 200, True, True), (2, 6, 12, 4, 8, 64, 12, False, True),
    (4, 80, 56, 32, 24, 96, 64, True, False), (3, 10, 12, 4, 8, 96, 64, True, False),    # key rows only
    (5, 7, 200, 56, 6, 320, 256, True, False), (2, 6, 100, 8, 8, 160, 128, False, False)])
def test_latent_prep(H, qlr, lat, rope, nope, D, off, own, vals, dt):
    torch.manual_seed(4)
    T, P = 11, 16
    a = torch.randn(T, qlr + (lat + rope if own else 0)).to(dt)
    w, pos, cs = (torch.rand(lat) + 0.5).to(dt), torch.randint(0, 100, (T,), dtype=torch.int32), torch.randn(128, rope)
    slots = torch.randperm(5 * P)[:T].to(torch.int32)
    slots[3] = -1                                        # a padding row lands in the scratch page
    q = torch.randn(T, H, nope + rope).to(dt)
    kc, vc, qf = torch.zeros(5, 1, P, D, dtype=dt), torch.zeros(5, 1, D, P, dtype=dt), torch.full((T, H, D), 7.0, dtype=dt)
    ref.latent_prep(a, qlr, lat, rope, w, 1e-6, pos, cs, slots, kc if own else None, vc if own and vals else None, q,
                    nope, qf, off)
    kc2, vc2, qf2 = torch.zeros_like(kc).to(DEV), torch.zeros_like(vc).to(DEV), torch.full((T, H, D), 7.0, dtype=dt).to(DEV)
    ops.latent_prep(a.to(DEV), qlr, lat, rope, w.to(DEV), 1e-6, pos.to(DEV), cs.to(DEV), slots.to(DEV),
                    kc2 if own else None, vc2 if own and vals else None, q.to(DEV), nope, qf2, rope_off=off)
    assert _close(kc2, kc, _tol(dt)) and _close(vc2, vc, _tol(dt)) and _close(qf2[:, :, lat:], qf[:, :, lat:], _tol(dt))
    assert torch.equal(qf2[:, :, :lat].cpu(), qf[:, :, :lat])          # the latent columns are the caller's
    if own:
        assert kc[:, :, :, lat:off].abs().sum() == 0 and kc[:, :, :, :lat].abs().sum() > 0      # the gap stays zero


@pytest.mark.parametrize("shape", list(ops.LATENT_SHAPES))
@pytest.mark.parametrize("H", [4, 16, 19])
def test_latent_attn_kernel(shape, H):
    """The MFMA latent kernel (key rows that carry their values, sinks) against the reference: prompt
    chunks whose rows see different key counts, decode rows over long and short contexts (split-K
    partials and their merge), partial pages, scattered block tables."""
    DK, DV = shape
    torch.manual_seed(DK + H)
    P, n_pages = 16, 200
    cache = (torch.randn(n_pages, P, DK, device=DEV) * 0.5).to(BF)
    sinks = torch.randn(H, device=DEV)
    kv_lens, q_lens = [3, 40, 1300, 97, 1], [3, 9, 20, 1, 1]
    bt = torch.stack([torch.randperm(n_pages - 1, device=DEV)[:84] + 1 for _ in kv_lens]).to(torch.int32)
    tok_row = torch.tensor([i for i, n in enumerate(q_lens) for _ in range(n)], dtype=torch.int32, device=DEV)
    tok_len = torch.tensor([kv - n + j + 1 for kv, n in zip(kv_lens, q_lens) for j in range(n)], dtype=torch.int32,
                           device=DEV)
    q = (torch.randn(int(tok_row.numel()), H, DK, device=DEV) * 0.5).to(BF)
    for sk in (sinks, None):
        got = ops.latent_attn(q, cache, bt, tok_row, tok_len, 0.15, DV, sinks=sk)
        want = ref.mla_attn(q.cpu(), cache.cpu(), bt.cpu(), tok_row.cpu(), tok_len.cpu(), 0.15, DV,
                            None if sk is None else sk.cpu())
        assert _close(got, want, 2e-2)
    qd = (torch.randn(5, H, DK, device=DEV) * 0.5).to(BF)                 # decode: one row per sequence
    rows = torch.arange(5, dtype=torch.int32, device=DEV)
    kl = torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
    got = ops.latent_attn(qd, cache, bt, rows, kl, 0.15, DV, sinks=sinks)
    want = ref.mla_attn(qd.cpu(), cache.cpu(), bt.cpu(), rows.cpu(), kl.cpu(), 0.15, DV, sinks.cpu())
    assert _close(got, want, 2e-2)


@pytest.mark.parametrize("Hq,D", [(4, 128), (6, 64), (16, 256), (5, 128)])
def test_float32_attention_with_sinks(Hq, D):
    torch.manual_seed(8)
    P, n_pages = 16, 90
    kc, vc = torch.randn(n_pages, 1, P, D, device=DEV), torch.randn(n_pages, 1, D, P, device=DEV)
    sinks = torch.randn(Hq, device=DEV) * 2
    kv_lens, q_lens = [3, 40, 1300, 97], [3, 9, 20, 1]
    bt = torch.stack([torch.randperm(n_pages - 1, device=DEV)[:84] + 1 for _ in kv_lens]).to(torch.int32)
    q = torch.randn(sum(q_lens), Hq, D, device=DEV)
    cu = torch.tensor([0, 3, 12, 32, 33], dtype=torch.int32, device=DEV)
    kl = torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
    items = torch.tensor(ops.prefill_work_items(q_lens, kv_lens), dtype=torch.int32, device=DEV)
    got = ops.paged_prefill(q, kc, vc, bt, cu, kl, items, 0.1, sinks=sinks)
    want = ref.paged_prefill(q.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), cu.cpu(), kl.cpu(), 0.1, sinks=sinks.cpu())
    assert (got.cpu() - want).abs().max().item() < 2e-5
    none = ref.paged_prefill(q.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), cu.cpu(), kl.cpu(), 0.1)
    assert (none - want).abs().max().item() > 0.05                    # the sinks matter
    qd = torch.randn(4, Hq, D, device=DEV)
    got = ops.paged_decode(qd, kc, vc, bt, kl, 0.1, None, sinks=sinks)
    want = ref.paged_decode(qd.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), kl.cpu(), 0.1, sinks=sinks.cpu())
    assert (got.cpu() - want).abs().max().item() < 2e-5


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("kw", [dict(), dict(heads=1, dim=8, rot_dim=8, vdim=8, kv_rank=8, q_rank=8, scaling=None),
                                dict(heads=5, dim=4, rot_dim=2, vdim=9, kv_rank=70, q_rank=5, base=5000.0, scale=0.5),
                                dict(heads=18, dim=4, rot_dim=4, vdim=2, kv_rank=6, q_rank=4),
                                dict(heads=4, dim=32, rot_dim=16, vdim=48, kv_rank=192, q_rank=80, scale=0.2)])
def test_latent_attention_alone(kw, dt):
    L = mo.attention_layer(**kw)
    cfg = mo.make_config([L], width=24)
    w, m = mo.sub(mo.random_weights(cfg, 3), "l0.mix."), L["mixer"]
    h = torch.randn(45, 24, generator=torch.Generator().manual_seed(3))
    want = mo.latent_attention(h.to(dt).to(F64), {k: v.to(F64) for k, v in w.items()}, m, 1e-5)
    for cuts in ([45], [40] + [1] * 5, [2, 3, 17, 16, 1, 6]):
        blk, kv = mc.attention_block(m, 24, DEV, dt)
        blk.load(w)
        assert _rel(mc.run_chunks(blk, h.to(device=DEV, dtype=dt), cuts, kv), want) < (0.04 if dt == BF else 1e-4), cuts


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("n,i,j", [(300, 299, 3), (300, 299, 0), (65, 64, 15), (65, 64, 16), (65, 64, 63), (40, 33, 32)])
@pytest.mark.parametrize("mode", ["whole", "decode", "portions"])
def test_planted_key_is_seen(n, i, j, mode, dt):
    cuts = {"whole": [n], "decode": [i] + [1] * (n - i), "portions": mc.portions(n, [2, 15, 1, 31, 16])}[mode]
    mc.planted_key_case(DEV, dt, 0.04 if dt == BF else 1e-4, n, i, j, cuts, row_only=dt == BF)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("cuts", [[40], [30, 10], [33, 2, 5]])
def test_future_key_is_not_seen(cuts, dt):
    mc.planted_key_case(DEV, dt, 0.04 if dt == BF else 1e-4, 40, 33, 34, cuts, seen=False, row_only=dt == BF)


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("m", [dict(heads=2, dim=6, vdim=10), dict(heads=1, dim=8, vdim=8), dict(heads=3, dim=20, vdim=3),
                               dict(heads=2, dim=64, vdim=64)])
def test_hgrn2_alone(m, dt):
    L = mo.hgrn2_layer(**m)
    w = mo.sub(mo.random_weights(mo.make_config([L], width=24), 4), "l0.mix.")
    h = torch.randn(37, 24, generator=torch.Generator().manual_seed(2))
    blk = Hgrn2Mixer(24, m["heads"], m["dim"], m["vdim"], 1e-5, DEV, dt)
    blk.load(w)
    want = mo.hgrn2(h.to(dt).to(F64), {k: v.to(F64) for k, v in w.items()}, m, 1e-5)
    for cuts in ([37], [1] * 37, [3, 2, 1, 9, 22]):
        assert _rel(mc.run_chunks(blk, h.to(device=DEV, dtype=dt), cuts), want) < (0.04 if dt == BF else 1e-4), cuts


@pytest.mark.parametrize("dt", DTYPES)
@pytest.mark.parametrize("f,width", [(mo.moe(5, 2, 12, 20), 24), (mo.moe(3, 1, 9, 0), 24), (mo.moe(4, 4, 8, 8), 24),
                                     (mo.moe(10, 1, 64, 96), 64), (mo.moe(6, 3, 32, 0), 96)])
def test_input_scaled_moe_alone(f, width, dt):
    """Both paths: the grouped GEMMs (bf16, widths in multiples of 32) and the batched dense one."""
    w = mo.sub(mo.random_weights(mo.make_config([mo.hgrn2_layer(mlp=f)], width=width), 9), "l0.mlp.")
    w64 = {k: v.to(F64) for k, v in w.items()}
    for seed in range(7, 300):     # inputs whose router decisions are clear of ties (the router sees the same
        h = torch.randn(13, width, generator=torch.Generator().manual_seed(seed))   # rounded rows as the oracle)
        if mo.router_margin(h.to(dt).to(F64), w64, f) > (2e-3 if dt == BF else 1e-4):
            break
    else:
        raise AssertionError("no input with the wanted router margin")
    blk = InputScaledMoE(width, f["router"]["experts"], f["router"]["top"], f["expert"]["ff"],
                         (f.get("shared") or {}).get("ff", 0), DEV, dt)
    blk.load(w)
    hd = h.to(device=DEV, dtype=dt)
    assert blk.grouped_ok(hd) == (dt == BF and width % 32 == 0 and f["expert"]["ff"] % 32 == 0)
    assert _rel(blk.forward(hd), mo.moe_ff(h.to(dt).to(F64), w64, f)) < (0.04 if dt == BF else 1e-4)


@pytest.mark.parametrize("dt", DTYPES)
def test_polynorm_mlp_alone(dt):
    w = mo.sub(mo.random_weights(mo.make_config([mo.hgrn2_layer(mlp=mo.dense(40))]), 8), "l0.mlp.")
    h = torch.randn(9, 24, generator=torch.Generator().manual_seed(6)) * 3
    blk = PolyNormMLP(24, 40, 1e-5, DEV, dt)
    blk.load(w)
    want = mo.polynorm_ff(h.to(dt).to(F64), {k: v.to(F64) for k, v in w.items()}, 1e-5)
    assert _rel(blk.forward(h.to(device=DEV, dtype=dt)), want) < (0.04 if dt == BF else 1e-4)


# ------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", mc.config_a()), ("b", mc.config_b()), ("c", mc.config_c()), ("h", mc.config_bf16())):
        w = mo.random_weights(cfg, seed=11, gain=0.5 if name == "h" else 1.0)
        out[name] = (cfg, w, mo.save_model(tmp_path_factory.mktemp("met_" + name), cfg, w), {})
    return out


def _schedules(toks):
    return (mc.whole_schedule(toks), mc.decode_schedule(toks, 24), mc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
            mc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31]))


@pytest.mark.parametrize("name", ["a", "b", "c"])
def test_float32_schedules_match_oracle(models, name):
    """A model served in float32 on the GPU: every schedule within fp32 rounding of the oracle."""
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", mc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=1e-4, cache=cache)))
    eng = mc.make_engine(path, DEV, "float32", max_tokens=192)
    for sched in _schedules(toks):
        mc.assert_matches_oracle(eng, cfg, w, toks, sched, 2e-4, cache)
    assert eng.runner.launch_stats["decode-graph"] > 0


def test_bfloat16_schedules_match_oracle(models):
    cfg, w, path, cache = models["h"]
    toks = dict(zip("pqrstu", mc.prompts(cfg, w, [1, 2, 37, 70, 16, 33], min_margin=0.02, cache=cache)))
    outs = []
    for sched in _schedules(toks):
        eng = mc.make_engine(path, DEV, "bfloat16", max_tokens=192)
        mc.assert_matches_oracle(eng, cfg, w, toks, sched, TOL, cache, TYPICAL)
        outs.append(mc.replay(mc.make_engine(path, DEV, "bfloat16", max_tokens=192), toks, sched))
    for o in outs[1:]:          # the same tokens under another schedule: only summation orders differ
        errs = torch.cat([mo.logit_errors(o[rid], outs[0][rid].double()) for rid in toks])
        assert errs.max().item() < TOL and errs.median().item() < 0.02


def test_slots_and_pages_are_reused(models):
    cfg, w, path, cache = models["h"]
    ps = mc.prompts(cfg, w, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25, 16, 30], seed=5, min_margin=0.02, cache=cache)
    toks = {f"r{i}": t for i, t in enumerate(ps)}
    for dt, tol, typ in (("bfloat16", TOL, TYPICAL), ("float32", 2e-4, None)):
        eng = mc.make_engine(path, DEV, dt, max_tokens=160)
        mc.assert_matches_oracle(eng, cfg, w, toks, mc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), tol, cache, typ)
        assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_graph_and_eager_decode_agree(models):
    cfg, w, path, cache = models["h"]
    toks = {"x": mc.prompts(cfg, w, [100], seed=9, min_margin=0.02, cache=cache)[0]}
    outs = []
    for graphs in (True, False):
        eng = mc.make_engine(path, DEV, "bfloat16", max_tokens=128, graphs=graphs)
        outs.append(mc.replay(eng, toks, mc.decode_schedule(toks, 95))["x"])
        errs = mo.logit_errors(outs[-1], cache[tuple(toks["x"])])
        assert errs.max().item() < TOL and errs.median().item() < TYPICAL
        assert eng.runner.launch_stats["decode-graph"] > 0 if graphs else not eng.runner.launch_stats["decode-graph"]
    errs = mo.logit_errors(outs[0], outs[1].double())
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
