"""Scenarios shared by the CPU (fp32 reference ops) and GPU (HIP kernels) Metitar tests: small
random models run through the engine's replay entry under different schedules, every position's
logits compared with the slow oracle of ``metitar_oracle``; single mixers run in portions; planted
keys.  The schedule builders are the ones of ``zavilorn_cases`` (they know nothing of a design)."""
from __future__ import annotations

import random

import torch

import metitar_oracle as mo
from ome_amd.models.common import AttnMeta, PagedKVCache
from ome_amd.models.mixers import LatentAttention, MixerCtx
from zavilorn_cases import (chunked_schedule, decode_schedule, greedy_engine, make_engine, mixed_schedule,  # noqa: F401
                            portions, replay, whole_schedule)

F64 = torch.float64


def config_a():
    """Attention first (its cache is read again by layer 3), two HGRN2 layers, dense and routed
    feed-forwards, one layer without a feed-forward; sizes that are all different from each other."""
    return mo.make_config([
        mo.attention_layer(mlp=mo.dense(40)),
        mo.hgrn2_layer(mlp=mo.moe(5, 2, 12, 20)),
        mo.hgrn2_layer(heads=3, dim=4, vdim=5, mlp=None),
        mo.attention_layer(heads=2, dim=6, vdim=10, q_rank=7, kv_from=0, scale=0.7, mlp=mo.moe(3, 1, 9, 0)),
    ])


def config_b():
    """Other sizes and the values the first config keeps apart made equal, 1 or absent: HGRN2
    first, dim = vdim = rot_dim, one head, two taps, no rotary scaling, every expert chosen (top =
    experts), no shared expert, unit logit scale, two attention layers with caches of their own and
    different widths, one of them read by a third."""
    return mo.make_config([
        mo.hgrn2_layer(heads=1, dim=8, vdim=8, mlp=mo.dense(17)),
        mo.attention_layer(heads=1, dim=8, rot_dim=8, vdim=8, kv_rank=8, q_rank=8, base=7.0, scaling=None, scale=1.0,
                           mlp=mo.moe(2, 2, 8, 0)),
        mo.attention_layer(heads=5, dim=4, rot_dim=2, vdim=3, kv_rank=70, q_rank=5, base=5000.0,
                           scaling={"factor": 2.0, "original": 8, "fast": 2.0, "slow": 0.5}, scale=0.3,
                           mlp=mo.dense(33)),
        mo.attention_layer(heads=2, dim=8, rot_dim=8, vdim=4, kv_rank=8, q_rank=3, base=7.0, scaling=None, scale=0.5,
                           kv_from=1, mlp=None),
    ], width=40, vocab=37, embed_scale=2.0, eps=1e-6, taps=2, side=2, logit_scale=1.0)


def config_c():
    """No input convolution, no per-layer token input, a single-tap-free stack of one attention and
    one HGRN2 layer (the optional parts absent)."""
    return mo.make_config([mo.attention_layer(mlp=mo.dense(16)), mo.hgrn2_layer(mlp=mo.moe(4, 1, 8, 8))],
                          width=16, vocab=29, taps=0, side=0)


def config_bf16():
    """For 16-bit runs: few routed evaluations with a wide router margin (two experts, one chosen)."""
    return mo.make_config([
        mo.attention_layer(heads=4, dim=16, rot_dim=8, vdim=12, kv_rank=24, q_rank=20, mlp=mo.dense(48)),
        mo.hgrn2_layer(heads=2, dim=16, vdim=8, mlp=mo.dense(40)),
        mo.attention_layer(heads=2, dim=8, rot_dim=8, vdim=16, kv_rank=24, q_rank=12, kv_from=0, mlp=mo.moe(2, 1, 32, 32)),
        mo.hgrn2_layer(heads=3, dim=8, vdim=24, mlp=None),
    ], width=64, vocab=61, taps=4, side=8, embed_scale=8.0)


def prompts(cfg, weights, lengths, seed=1, min_margin=0.0, cache=None):
    """Random prompts; with ``min_margin`` > 0 each prompt's seed is advanced until every router
    decision on it has at least that margin in the oracle (a 16-bit run may otherwise pick another
    expert on a near tie, which is no fault).  Oracle logits land in ``cache``."""
    out = []
    for k, n in enumerate(lengths):
        for s in range(200):
            g = random.Random(1000 * (seed + s) + k)
            p = [g.randrange(cfg["vocab"]) for _ in range(n)]
            m: list = []
            want = mo.forward(cfg, weights, p, margins=m)
            if not m or min(m) >= min_margin:
                if cache is not None:
                    cache[tuple(p)] = want
                out.append(p)
                break
        else:
            raise AssertionError("no prompt with the wanted router margin")
    return out


def assert_matches_oracle(eng, cfg, weights, toks: dict, schedule, tol, oracle_cache=None, typical=None):
    """Every position within ``tol`` of the oracle.  ``typical`` (16-bit runs): also the median over
    all positions -- the design's output norms amplify 16-bit rounding at single positions of a small
    random model, while a fault of the cache, the state or a mask moves most positions by far more."""
    got = replay(eng, toks, schedule)
    worst, every = 0.0, []
    for rid, t in toks.items():
        key = tuple(t)
        if oracle_cache is not None and key in oracle_cache:
            want = oracle_cache[key]
        else:
            want = mo.forward(cfg, weights, t)
            if oracle_cache is not None:
                oracle_cache[key] = want
        errs = mo.logit_errors(got[rid], want)
        every.append(errs)
        err = errs.max().item()
        worst = max(worst, err)
        assert err < tol, f"request {rid} ({len(t)} tokens): logits differ from the oracle by {err:.3g} (limit {tol})"
    if typical is not None:
        med = torch.cat(every).median().item()
        assert med < typical, f"median difference from the oracle {med:.3g} (limit {typical})"
    return worst


def greedy_reference(cfg, weights, prompt, n):
    """n greedy tokens from the oracle; also the smallest top-1 / top-2 logit gap met on the way."""
    t, gap = list(prompt), float("inf")
    for _ in range(n):
        lg = mo.forward(cfg, weights, t)[-1]
        top = torch.topk(lg, 2).values
        gap = min(gap, float(top[0] - top[1]))
        t.append(int(lg.argmax()))
    return t[len(prompt):], gap


# ------------------------------------------------------------------------------ one mixer alone
def run_chunks(block, h, cuts, kv=None, page=16, slot=1, first_page=7):
    """One sequence through ``block`` in portions ``cuts`` (state slot ``slot``, a scattered page
    table); single rows go as decode steps, longer portions as prompt chunks."""
    T = h.shape[0]
    n_pages = -(-T // page)
    dev = h.device
    table = torch.tensor([[first_page + 2 * i for i in range(n_pages)]], dtype=torch.int32, device=dev)
    block.alloc_state(slot + 2)
    i32 = dict(dtype=torch.int32, device=dev)
    outs, a = [], 0
    for n in cuts:
        pos = torch.arange(a, a + n, **i32)
        slots = (table[0, (pos // page).long()] * page + pos % page).to(torch.int32)
        if n == 1 and a > 0:
            meta = AttnMeta("decode", pos, slots, table, seq_lens=torch.tensor([a + 1], **i32))
        else:
            meta = AttnMeta("prefill", pos, slots, table, cu_q=torch.tensor([0, n], **i32),
                            kv_lens=torch.tensor([a + n], **i32),
                            items=torch.tensor([[0, r] for r in range(0, n, 32)], **i32))
        seqs = (torch.tensor([0, n], **i32), torch.tensor([slot], **i32), torch.tensor([int(a == 0)], **i32))
        outs.append(block.forward(h[a:a + n].contiguous(), MixerCtx(meta, kv, seqs)))
        a += n
    return torch.cat(outs)


def attention_block(m, width, dev, dt, eps=1e-5, max_pos=512, pages=96):
    blk = LatentAttention(0, 0, width, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"],
                          m["rot"]["base"], m["rot"].get("scaling"), m["scale"], eps, max_pos, dev, dt)
    return blk, PagedKVCache(1, pages, 1, blk.D, 16, dt, dev)


def planted_key_case(dev, dt, tol, n, i, j, cuts, seen=True, row_only=False):
    """A key made to dominate query i's softmax whenever it is visible.  The latent's first half
    reads the input's first half and feeds the keys, its second half reads the input's second half
    and feeds the values; q's unrotated part is tied to k's (same down projection, norm weight and
    up projection) and nothing rotated reaches the score, so a row j that repeats row i's first
    half has the query's own key direction but a value of its own; its second half is small, which
    makes its normalised latent (and so its score) larger than the query's own.  Losing (or wrongly
    seeing) that one key among hundreds moves the output by much more than the tolerance.
    ``seen`` False: j > i lies in the future of query i and must leave its output alone.
    ``row_only``: compare row i alone (16-bit runs: the other rows' softmaxes are as sharp but
    between random keys, where rounding of the scores decides)."""
    W, R, r, d = 64, 32, 4, 32
    m = mo.attention_layer(heads=2, dim=d, rot_dim=r, vdim=8, kv_rank=R, q_rank=R, scale=0.5)["mixer"]
    w = mo.sub(mo.random_weights(mo.make_config([{"type": "latent_attention", "mixer": m, "mlp": None}], width=W), 21),
               "l0.mix.")
    half = W // 2
    w["dkv"][:R // 2, half:] = 0          # latent first half <- input first half
    w["dkv"][R // 2:R, :half] = 0         # latent second half <- input second half
    w["dq"] = w["dkv"][:R].clone()
    w["dq.norm"] = w["dkv.norm"].clone()
    w["uk"][:, R // 2:] = 0               # keys read the first half of the latent,
    w["uv"][:, :R // 2] = 0               # values the second
    uq = w["uq"].view(2, d + r, R)
    uq[:, :d] = w["uk"].view(2, d, R)
    uq[:, d:] = 0                         # no rotated part in the score
    w["sink"] = torch.full((2,), -4.0, dtype=torch.bfloat16)
    h = torch.randn(n, W, generator=torch.Generator().manual_seed(8))
    h[j, :half] = h[i, :half]
    h[j, half:] *= 0.3
    w64 = {k: v.to(F64) for k, v in w.items()}
    hq = h.to(dt).to(F64)
    want = mo.latent_attention(hq, w64, m, 1e-5)
    blk, kv = attention_block(m, W, dev, dt, pages=2 * (n // 16 + 2) + 8)
    blk.load(w)
    got = run_chunks(blk, h.to(device=dev, dtype=dt), cuts, kv).cpu()
    rows = slice(i, i + 1) if row_only else slice(None)
    rel = ((got.to(F64) - want)[rows].abs().max() / want[rows].abs().max()).item()
    assert rel < tol, rel
    if seen:    # the planted key carries the answer: hidden, the oracle's row i moves
        moved = mo.latent_attention(hq, w64, m, 1e-5, hide=(i, j))
    else:       # seen by mistake it would: compare with the oracle run on a row order where j comes first
        perm = list(range(n))
        perm[j], perm[i - 1] = perm[i - 1], perm[j]
        moved = mo.latent_attention(hq[perm], w64, m, 1e-5)
    assert (moved[i] - want[i]).abs().max() > 0.08 * want[i].abs().max()
