"""Zavilorn on gfx950: the HIP kernels added for it against their fp32 references (odd sizes and
unaligned views included), then whole bf16 models through the engine (HIP-graph decode, eager
mixed steps) against the slow fp64 oracle under the same schedules as the CPU tests."""
import os
import sys

import pytest
import torch

sys.path.insert(0, os.path.dirname(os.path.abspath(__file__)))

import zavilorn_cases as zc  # noqa: E402
import zavilorn_oracle as zo  # noqa: E402
from ome_amd import ops  # noqa: E402
from ome_amd.ops import reference as ref  # noqa: E402

pytestmark = pytest.mark.gpu
DEV = "cuda"
BF = torch.bfloat16
TOL = 0.08     # bf16 projections / activations against an fp64 oracle (the CPU bf16 path is ~0.03 off)
SAME = 0.04    # the same tokens under another schedule: only summation orders differ


def _close(got, want, tol):
    want = want.float()
    if want.numel() == 0:
        return got.shape == want.shape
    return (got.float().cpu() - want).abs().max().item() <= tol * max(1.0, want.abs().max().item())


@pytest.mark.parametrize("T,H", [(1, 48), (37, 256), (5, 1000)])
@pytest.mark.parametrize("n_add", [0, 1, 2])
def test_residual_rmsnorm(T, H, n_add):
    torch.manual_seed(0)
    res = torch.randn(T, H, device=DEV) * 4
    w = (torch.rand(H, device=DEV) + 0.5).to(BF)
    x1 = torch.randn(T, H, device=DEV).to(BF) if n_add >= 1 else None
    x2 = torch.randn(T, H + 3, device=DEV).to(BF)[:, 3:] if n_add == 2 else None
    r_ref = res.cpu().clone()
    want = ref.residual_rmsnorm(r_ref, w.cpu(), 1e-6, None if x1 is None else x1.cpu(), 0.6,
                                None if x2 is None else x2.cpu(), 0.5)
    got = ops.residual_rmsnorm(res, w, 1e-6, x1, 0.6, x2, 0.5)
    assert got.dtype == BF and _close(got, want, 1e-2)
    assert (res.cpu() - r_ref).abs().max().item() < 1e-5


def test_embedding_f32_and_lm_head():
    torch.manual_seed(0)
    table = torch.randn(61, 40, device=DEV).to(BF)
    ids = torch.tensor([0, 60, 7, 7, 33], dtype=torch.int32, device=DEV)
    got = ops.embedding_f32(ids, table, 4.0)
    assert got.dtype == torch.float32 and torch.equal(got.cpu(), table.cpu().float()[ids.cpu().long()] * 4.0)
    h = torch.randn(5, 40, device=DEV).to(BF)
    lg = ops.lm_head_f32(h, table)
    assert lg.dtype == torch.float32
    assert (lg.cpu() - h.cpu().float() @ table.cpu().float().T).abs().max().item() < 1e-3


@pytest.mark.parametrize("pad", [5, 0])   # 0: rows and segments 16-byte aligned (the vector kernel where it applies)
@pytest.mark.parametrize("Hq,Hkv,dim,vdim,rot,inter", [(6, 2, 80, 72, 40, True), (2, 2, 8, 12, 8, True),
                                                         (4, 2, 70, 36, 2, True), (3, 1, 64, 64, 32, False),
                                                         (2, 1, 24, 16, 0, True), (8, 2, 128, 128, 64, True),
                                                         (4, 2, 64, 32, 10, True)])
def test_wide_norm_rope_cache(Hq, Hkv, dim, vdim, rot, inter, pad):
    torch.manual_seed(1)
    from ome_amd.models.config import attn_tile_dim, plain_rope_table

    T, P, D = 21, 16, attn_tile_dim(max(dim, vdim))
    nq, nk, nv = Hq * dim, Hkv * dim, Hkv * vdim
    p = torch.randn(T, nq + nk + nv + pad, device=DEV).to(BF)
    q, k, v = p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:nq + nk + nv]
    qw, kw = (torch.rand(nq, device=DEV) + 0.5).to(BF), (torch.rand(nk, device=DEV) + 0.5).to(BF)
    cs = plain_rope_table(3000.0, rot, 400, DEV) if rot else torch.zeros(400, 0, device=DEV)
    pos = torch.randint(0, 400, (T,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(5 * P, device=DEV)[:T].to(torch.int32) + P
    slots[3] = -1
    outs = []
    for dev in (DEV, "cpu"):
        kc = torch.zeros(8, Hkv, P, D, dtype=BF, device=dev)
        vc = torch.zeros(8, Hkv, D, P, dtype=BF, device=dev)
        qo = torch.full((T, Hq, D), 9.0, dtype=BF, device=dev)
        mv = (lambda t: t) if dev == DEV else (lambda t: t.cpu())
        ops.wide_norm_rope_cache(mv(q), mv(k), mv(v), mv(pos), mv(cs), rot, inter, mv(qw), mv(kw), 1e-6, qo, kc, vc,
                                 mv(slots), Hq, Hkv, dim, vdim)
        outs.append((qo, kc, vc))
    for g, w in zip(*outs):
        assert _close(g, w, 2e-2)
    assert outs[0][0][:, :, dim:].abs().max().item() == 0 if dim < D else True


def test_head_gate_and_clamped_glu():
    torch.manual_seed(2)
    T, H, D, vd = 9, 3, 64, 36
    o = torch.randn(T, H, D, device=DEV).to(BF)
    g = torch.randn(T, H * vd + 7, device=DEV).to(BF)[:, 7:]
    for kind in (0, 1):
        assert _close(ops.head_gate(o, g, vd, kind), ref.head_gate(o.cpu(), g.cpu(), vd, kind), 1e-2)
    for I, lim in ((352, 2.5), (13, 0.5), (64, 0.0)):
        x = (torch.randn(T, 2 * I, device=DEV) * 3).to(BF)
        assert _close(ops.act_and_mul(x, 2, limit=lim), ref.act_and_mul(x.cpu(), 2, lim), 1e-2)


@pytest.mark.parametrize("H,P,N,G,pad", [(6, 32, 24, 3, 4), (3, 5, 7, 3, 1), (2, 64, 128, 1, 0), (4, 64, 128, 2, 3),
                                         (1, 16, 8, 1, 0)])
def test_ssm_scan_any_shape(H, P, N, G, pad):
    torch.manual_seed(3)
    lens = [6, 1, 33]
    T, I, GN = sum(lens), H * P, G * N
    buf = torch.randn(T, I + 2 * GN + H + pad, device=DEV).to(BF)
    x, B, C, dt = buf[:, :I], buf[:, I:I + GN], buf[:, I + GN:I + 2 * GN], buf[:, I + 2 * GN:I + 2 * GN + H]
    A = -torch.rand(H, device=DEV) * 2 - 0.1
    Dp, dtb = torch.rand(H, device=DEV) + 0.5, torch.randn(H, device=DEV)
    cu = torch.tensor([0, 6, 7, 40], dtype=torch.int32, device=DEV)
    slot = torch.tensor([2, 0, 3], dtype=torch.int32, device=DEV)
    reset = torch.tensor([1, 0, 0], dtype=torch.int32, device=DEV)
    st0 = torch.randn(4, H, P, N, device=DEV) * 0.2
    st_k, st_r = st0.clone(), st0.cpu().clone()
    y = ops.ssm_scan(x, dt, B, C, A, Dp, dtb, 0.0, st_k, cu, slot, reset, H, P, N, G)
    c = lambda t: t.cpu()  # noqa: E731
    yr = ref.ssm_scan(c(x), c(dt), c(B), c(C), c(A), c(Dp), c(dtb), 0.0, st_r, c(cu), c(slot), c(reset), H, P, N, G,
                      torch.empty(T, I, dtype=BF))
    assert _close(y, yr, 2e-2)
    assert (st_k.cpu() - st_r).abs().max().item() < 1e-3 * max(1.0, st_r.abs().max().item())
    assert torch.equal(st_k[1].cpu(), st0[1].cpu())


@pytest.mark.parametrize("dk,dv,Hk,Hv,pad", [(32, 48, 2, 6, 0), (5, 4, 3, 3, 1), (12, 20, 1, 2, 3), (10, 4, 1, 3, 0),
                                             (96, 160, 1, 2, 0)])
def test_gdn_scan_any_shape(dk, dv, Hk, Hv, pad):
    torch.manual_seed(4)
    lens = [5, 1, 40]
    T, kd, vd = sum(lens), Hk * dk, Hv * dv
    proj = torch.randn(T, 2 * kd + vd + 2 * Hv + pad, device=DEV).to(BF)
    q, k, v = proj[:, :kd], proj[:, kd:2 * kd], proj[:, 2 * kd:2 * kd + vd]
    b, a = proj[:, 2 * kd + vd:2 * kd + vd + Hv], proj[:, 2 * kd + vd + Hv:2 * kd + vd + 2 * Hv]
    A_log, dtb = torch.rand(Hv, device=DEV) * 2 - 1, torch.randn(Hv, device=DEV) * 0.5
    cu = torch.tensor([0, 5, 6, 46], dtype=torch.int32, device=DEV)
    slot = torch.tensor([2, 0, 3], dtype=torch.int32, device=DEV)
    reset = torch.tensor([1, 0, 0], dtype=torch.int32, device=DEV)
    st0 = torch.randn(4, Hv, dv, dk, device=DEV) * 0.1
    st_k, st_r = st0.clone(), st0.cpu().clone()
    y = ops.gdn_scan(q, k, v, a, b, A_log, dtb, st_k, cu, slot, reset, Hv, Hk)
    c = lambda t: t.cpu()  # noqa: E731
    yr = ref.gdn_scan(c(q), c(k), c(v), c(a), c(b), c(A_log), c(dtb), st_r, c(cu), c(slot), c(reset), Hv, Hk,
                      torch.empty(T, vd, dtype=BF))
    assert _close(y, yr, 2e-2)
    assert (st_k.cpu() - st_r).abs().max().item() < 1e-3 * max(1.0, st_r.abs().max().item())
    assert torch.equal(st_k[1].cpu(), st0[1].cpu())


@pytest.mark.parametrize("K", [1, 3, 7, 9, 20])
def test_conv_any_taps(K):
    torch.manual_seed(5)
    C, lens = 37, [4, 1, 19]
    T = sum(lens)
    x = torch.randn(T, C + 3, device=DEV).to(BF)[:, 3:]
    w, bias = (torch.randn(C, K, device=DEV) * 0.5).to(BF), (torch.randn(C, device=DEV) * 0.1).to(BF)
    cu = torch.tensor([0, 4, 5, 24], dtype=torch.int32, device=DEV)
    slot = torch.tensor([1, 0, 2], dtype=torch.int32, device=DEV)
    reset = torch.tensor([1, 0, 0], dtype=torch.int32, device=DEV)
    st0 = torch.randn(3, C, K - 1, device=DEV).to(BF)
    st_k, st_r = st0.clone(), st0.cpu().clone()
    y = ops.ssm_conv1d(x, w, bias, st_k, cu, slot, reset)
    yr = ref.ssm_conv1d(x.cpu(), w.cpu(), bias.cpu(), st_r, cu.cpu(), slot.cpu(), reset.cpu(), torch.empty(T, C, dtype=BF))
    assert _close(y, yr, 2e-2) and _close(st_k, st_r, 1e-2)


@pytest.mark.parametrize("Hq,Hkv,D", [(4, 1, 128), (4, 2, 64), (8, 2, 128), (2, 2, 256)])
@pytest.mark.parametrize("window,keep", [(70, 6), (40, 33), (5, 1), (300, 7), (16, 0)])
def test_attention_kept_first_keys(Hq, Hkv, D, window, keep):
    """Prefill (prompt chunks over a prefix) and decode rows with a sliding window that keeps the
    first keys, against the reference mask; sequence lengths put the window's start before, at
    and after the kept range and across 32-key tile borders."""
    torch.manual_seed(6)
    P, n_pages = 16, 64
    kc = (torch.randn(n_pages, Hkv, P, D, device=DEV) * 0.5).to(BF)
    vc = (torch.randn(n_pages, Hkv, D, P, device=DEV) * 0.5).to(BF)
    kv_lens = [3, 40, 77, 130, 200, 97]
    q_lens = [3, 9, 77, 2, 33, 1]
    B = len(kv_lens)
    bt = torch.stack([torch.randperm(n_pages - 1, device=DEV)[:16] + 1 for _ in range(B)]).to(torch.int32)
    scale = 0.3
    # prefill
    Tq = sum(q_lens)
    q = torch.randn(Tq, Hq, D, device=DEV).to(BF)
    cu = torch.tensor([0] + list(torch.tensor(q_lens).cumsum(0)), dtype=torch.int32, device=DEV)
    kl = torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
    items = torch.tensor(ops.prefill_work_items(q_lens, kv_lens), dtype=torch.int32, device=DEV)
    got = ops.paged_prefill(q, kc, vc, bt, cu, kl, items, scale, window, keep_first=keep)
    want = ref.paged_prefill(q.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), cu.cpu(), kl.cpu(), scale, window, keep_first=keep)
    assert _close(got, want, 1e-2)
    # decode: one query per sequence at its last position
    qd = torch.randn(B, Hq, D, device=DEV).to(BF)
    for parts in (None, 3):
        ws = None if parts is None else ops.DecodeWorkspace(B, Hq, D, 16 * P, 0, DEV, parts=parts)
        got = ops.paged_decode(qd, kc, vc, bt, kl, scale, ws, window, keep_first=keep)
        want = ref.paged_decode(qd.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), kl.cpu(), scale, window, keep_first=keep)
        assert _close(got, want, 1e-2), parts


@pytest.mark.parametrize("gap,seen", [(8, True), (9, False)])
@pytest.mark.parametrize("cuts", [[60], [59, 1], [7, 2, 30, 21]])
def test_window_edge_shows(gap, seen, cuts):
    zc.planted_window_case(DEV, BF, 0.06, gap, seen, cuts)


@pytest.mark.parametrize("j,seen", [(2, True), (3, False)])
@pytest.mark.parametrize("cuts", [[50], [49, 1], [2, 2, 46]])
def test_kept_first_edge_shows(j, seen, cuts):
    zc.planted_kept_case(DEV, BF, 0.06, j, seen, cuts)


# ------------------------------------------------------------------------------ whole models
@pytest.fixture(scope="module")
def models(tmp_path_factory):
    out = {}
    for name, cfg in (("a", zc.config_a()), ("b", zc.config_b())):
        w = zo.random_weights(cfg, seed=11, gain=0.5)   # (gain 1 amplifies bf16 rounding to ~0.3)
        out[name] = (cfg, w, zo.save_model(tmp_path_factory.mktemp("zav_" + name), cfg, w), {})
    return out


@pytest.mark.parametrize("name", ["a", "b"])
def test_schedules_match_oracle(models, name):
    cfg, w, path, cache = models[name]
    toks = dict(zip("pqrstu", zc.prompts(cfg, [1, 2, 37, 70, 16, 33])))
    eng = zc.make_engine(path, DEV, "bfloat16", max_tokens=192)
    base = zc.replay(eng, toks, zc.whole_schedule(toks))
    for sched in (zc.whole_schedule(toks), zc.decode_schedule(toks, 24), zc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
                  zc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31])):
        zc.assert_matches_oracle(eng, cfg, w, toks, sched, TOL, cache)
        got = zc.replay(eng, toks, sched)
        for rid in toks:
            assert zo.logit_error(got[rid], base[rid].double()) < SAME, rid
    assert eng.runner.launch_stats["decode-graph"] > 0      # single-token steps replayed HIP graphs


def test_slots_and_pages_are_reused(models):
    cfg, w, path, cache = models["a"]
    toks = {f"r{i}": t for i, t in enumerate(zc.prompts(cfg, [20, 3, 41, 17, 2, 33, 9, 48, 1, 25, 16, 30], seed=5))}
    eng = zc.make_engine(path, DEV, "bfloat16", max_tokens=160)
    zc.assert_matches_oracle(eng, cfg, w, toks, zc.mixed_schedule(toks, [2, 7, 1, 16, 3], seed=8), TOL, cache)
    assert eng.runner.pages.num_free == eng.runner.pages.num_pages - 1 and not eng.scheduler.running


def test_graph_and_eager_decode_agree(models):
    cfg, w, path, cache = models["a"]
    toks = {"x": zc.prompts(cfg, [100], seed=9)[0]}
    outs = []
    for graphs in (True, False):
        eng = zc.make_engine(path, DEV, "bfloat16", max_tokens=128, graphs=graphs)
        outs.append(zc.replay(eng, toks, zc.decode_schedule(toks, 95))["x"])
        zc.assert_matches_oracle(eng, cfg, w, toks, zc.decode_schedule(toks, 95), TOL, cache)
    assert zo.logit_error(outs[0], outs[1].double()) < 1e-3


def test_greedy_generation(models):
    cfg, w, path, _ = models["a"]
    ps = zc.prompts(cfg, [5, 19, 1], seed=13)
    eng = zc.make_engine(path, DEV, "bfloat16", max_tokens=256)
    got = zc.greedy_engine(eng, ps, 12)
    for p, g in zip(ps, got):
        want, gap = zc.greedy_reference(cfg, w, p, 12)
        assert len(g) == 12
        if gap > 0.25:                      # bf16: only clear-cut argmaxes are pinned
            assert g == want


# ------------------------------------------------------------------------------ float32 serving
def test_float32_ops_match_reference():
    """The float instantiations of the kernels an fp32 model runs on, against the references."""
    torch.manual_seed(7)
    f = lambda *s: torch.randn(*s, device=DEV)  # noqa: E731
    c = lambda t: t.cpu()  # noqa: E731
    tight = lambda g, w: (g.cpu() - w).abs().max().item() <= 2e-5 * max(1.0, w.abs().max().item())  # noqa: E731
    # residual + norm, gate, clamped GLU, embedding
    res, x1, x2, w = f(9, 50) * 4, f(9, 50), f(9, 50), torch.rand(50, device=DEV) + 0.5
    r_ref = res.cpu().clone()
    assert tight(ops.residual_rmsnorm(res, w, 1e-6, x1, 0.6, x2, 0.5), ref.residual_rmsnorm(r_ref, c(w), 1e-6, c(x1),
                                                                                            0.6, c(x2), 0.5))
    o, g = f(7, 3, 64), f(7, 3 * 36)
    assert tight(ops.head_gate(o, g, 36, 0), ref.head_gate(c(o), c(g), 36, 0))
    x = f(7, 2 * 24) * 3
    assert tight(ops.act_and_mul(x, 2, limit=2.5), ref.act_and_mul(c(x), 2, 2.5))
    tab = f(11, 16)
    ids = torch.tensor([3, 0, 10], dtype=torch.int32, device=DEV)
    assert torch.equal(ops.embedding_f32(ids, tab, 2.0).cpu(), tab.cpu()[[3, 0, 10]] * 2.0)
    # conv, scans, gated norm
    cu = torch.tensor([0, 5, 6, 30], dtype=torch.int32, device=DEV)
    slot = torch.tensor([2, 0, 1], dtype=torch.int32, device=DEV)
    reset = torch.tensor([1, 0, 0], dtype=torch.int32, device=DEV)
    xc, wc, bc = f(30, 21), f(21, 4) * 0.5, f(21) * 0.1
    st = f(3, 21, 3)
    st_r = st.cpu().clone()
    yc = ops.ssm_conv1d(xc, wc, bc, st, cu, slot, reset)
    assert tight(yc, ref.ssm_conv1d(c(xc), c(wc), c(bc), st_r, c(cu), c(slot), c(reset), torch.empty(30, 21)))
    assert tight(st, st_r)
    H, P, N, G = 4, 6, 10, 2
    buf = f(30, H * P + 2 * G * N + H)
    xs, B, C, dt = buf[:, :H * P], buf[:, H * P:H * P + G * N], buf[:, H * P + G * N:H * P + 2 * G * N], buf[:, -H:]
    A, Dp, dtb = -torch.rand(H, device=DEV) - 0.1, torch.rand(H, device=DEV), f(H)
    s0 = f(3, H, P, N) * 0.2
    s_r = s0.cpu().clone()
    y = ops.ssm_scan(xs, dt, B, C, A, Dp, dtb, 0.0, s0, cu, slot, reset, H, P, N, G)
    assert tight(y, ref.ssm_scan(c(xs), c(dt), c(B), c(C), c(A), c(Dp), c(dtb), 0.0, s_r, c(cu), c(slot), c(reset), H, P,
                                 N, G, torch.empty(30, H * P)))
    assert tight(s0, s_r)
    Hv, Hk, dk, dv = 4, 2, 64, 12          # (dk 64: an fp32 model still takes the generic kernel)
    pr = f(30, 2 * Hk * dk + Hv * dv + 2 * Hv)
    q, k, v = pr[:, :Hk * dk], pr[:, Hk * dk:2 * Hk * dk], pr[:, 2 * Hk * dk:2 * Hk * dk + Hv * dv]
    b, a = pr[:, -2 * Hv:-Hv], pr[:, -Hv:]
    Al, db = torch.rand(Hv, device=DEV) - 0.5, f(Hv) * 0.5
    g0 = f(3, Hv, dv, dk) * 0.1
    g_r = g0.cpu().clone()
    yo = ops.gdn_scan(q, k, v, a, b, Al, db, g0, cu, slot, reset, Hv, Hk)
    assert tight(yo, ref.gdn_scan(c(q), c(k), c(v), c(a), c(b), c(Al), c(db), g_r, c(cu), c(slot), c(reset), Hv, Hk,
                                  torch.empty(30, Hv * dv)))
    assert tight(g0, g_r)
    yy, zz, ww = f(9, 48), f(9, 48), torch.rand(48, device=DEV) + 0.5
    for nf in (False, True):
        for ex in (False, True):
            wv = ww[:12].contiguous() if nf else ww
            assert tight(ops.gated_rmsnorm(yy, zz, wv, 12, 1e-6, norm_first=nf, exact=ex),
                         ref.gated_rmsnorm(c(yy), c(zz), c(wv), 12, 1e-6, nf, ex))
            yb, zb, wb = yy.to(BF), zz.to(BF), wv.to(BF)
            assert _close(ops.gated_rmsnorm(yb, zb, wb, 12, 1e-6, norm_first=nf, exact=ex),
                          ref.gated_rmsnorm(c(yb), c(zb), c(wb), 12, 1e-6, nf, ex), 1e-2)


@pytest.mark.parametrize("window,keep", [(-1, 0), (9, 3), (40, 0), (2000, 5)])
def test_float32_attention(window, keep):
    torch.manual_seed(8)
    Hq, Hkv, D, P, n_pages = 4, 2, 64, 16, 90
    kc, vc = torch.randn(n_pages, Hkv, P, D, device=DEV), torch.randn(n_pages, Hkv, D, P, device=DEV)
    kv_lens, q_lens = [3, 40, 1300, 97], [3, 9, 20, 1]
    bt = torch.stack([torch.randperm(n_pages - 1, device=DEV)[:84] + 1 for _ in kv_lens]).to(torch.int32)
    q = torch.randn(sum(q_lens), Hq, D, device=DEV)
    cu = torch.tensor([0, 3, 12, 32, 33], dtype=torch.int32, device=DEV)
    kl = torch.tensor(kv_lens, dtype=torch.int32, device=DEV)
    items = torch.tensor(ops.prefill_work_items(q_lens, kv_lens), dtype=torch.int32, device=DEV)
    got = ops.paged_prefill(q, kc, vc, bt, cu, kl, items, 0.2, window, keep_first=keep)
    want = ref.paged_prefill(q.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), cu.cpu(), kl.cpu(), 0.2, window, keep_first=keep)
    assert (got.cpu() - want).abs().max().item() < 2e-5
    qd = torch.randn(4, Hq, D, device=DEV)
    kl0 = torch.tensor([3, 0, 1300, 97], dtype=torch.int32, device=DEV)     # a padding row (length 0)
    got = ops.paged_decode(qd, kc, vc, bt, kl0, 0.2, None, window, keep_first=keep)
    want = ref.paged_decode(qd.cpu(), kc.cpu(), vc.cpu(), bt.cpu(), kl0.cpu(), 0.2, window, keep_first=keep)
    assert (got.cpu() - want).abs().max().item() < 2e-5


@pytest.mark.parametrize("name", ["a", "b"])
def test_float32_schedules_match_oracle(models, name):
    """A model served in float32 on the GPU: every schedule within fp32 rounding of the oracle."""
    cfg, _, _, _ = models[name]
    w = zo.random_weights(cfg, seed=11)
    import tempfile

    path = zo.save_model(tempfile.mkdtemp(), cfg, w)
    toks = dict(zip("pqrstu", zc.prompts(cfg, [1, 2, 37, 70, 16, 33])))
    cache = {}
    eng = zc.make_engine(path, DEV, "float32", max_tokens=192)
    for sched in (zc.whole_schedule(toks), zc.decode_schedule(toks, 24), zc.chunked_schedule(toks, [2, 3, 17, 1, 32, 2]),
                  zc.mixed_schedule(toks, [1, 2, 5, 16, 1, 31])):
        zc.assert_matches_oracle(eng, cfg, w, toks, sched, 2e-4, cache)
    assert eng.runner.launch_stats["decode-graph"] > 0
