"""Scenarios shared by the CPU (fp32 reference ops) and GPU (bf16 HIP kernels) Zavilorn tests:
small random models run through the engine's replay entry under different schedules, every
position's logits compared with the slow oracle of ``zavilorn_oracle``."""
from __future__ import annotations

import random

import torch

import zavilorn_oracle as zo
from ome_amd.models.common import AttnMeta, PagedKVCache
from ome_amd.models.mixers import GatedWindowAttention, MixerCtx
from ome_amd.runtime.engine import Engine, EngineArgs
from ome_amd.runtime.request import SamplingParams


def config_a():
    """Parallel block first, odd sizes, window 9 keeping 2 first tokens, two Mamba-2 layers."""
    return zo.make_config([zo.parallel_layer(), zo.mamba_layer(), zo.mamba_layer(heads=4, vdim=4, state=6, groups=2,
                                                                                 conv=3, norm_groups=1, ff=24)])


def config_b():
    """Other sizes: Mamba-2 first, values the first config makes unequal are equal or 1 here (kv
    heads = heads, keep_first 0, rotary over the whole head, vdim > dim, 2-tap convolutions, one
    norm group), two parallel blocks with different head widths / windows, no feed-forward on one."""
    return zo.make_config([
        zo.mamba_layer(heads=1, vdim=16, state=8, groups=1, conv=2, norm_groups=1, ff=32, limit=0.75),
        zo.parallel_layer(heads=2, kv_heads=2, dim=8, vdim=12, window=5, keep_first=0, rot_dims=8, rot_base=7.0,
                          r_heads=2, r_kv_heads=2, r_dim=6, r_vdim=6, r_conv=2, ff=0, left_scale=1.0,
                          right_scale=1.0),
        zo.parallel_layer(heads=4, kv_heads=2, dim=70, vdim=36, window=1000, keep_first=3, rot_dims=2,
                          rot_base=5000.0, r_heads=3, r_kv_heads=1, r_dim=10, r_vdim=4, r_conv=4, ff=56, limit=6.0),
    ], width=40, vocab=37, embed_scale=1.0, eps=1e-6)


def make_engine(path, device, dtype, max_tokens=256, graphs=True):
    return Engine(EngineArgs(model_path=path, dtype=dtype, device=device, load_format="safetensors",
                             max_running_requests=4, max_total_tokens=max_tokens, context_length=max_tokens,
                             page_size=16, cuda_graph=graphs, cuda_graph_max_bs=4, disable_radix_cache=True,
                             keep_logits=True, watchdog_timeout=0.0, overlap_schedule=False))


def prompts(cfg, lengths, seed=1):
    g = random.Random(seed)
    return [[g.randrange(cfg["vocab"]) for _ in range(n)] for n in lengths]


def replay(eng, toks: dict, schedule):
    """schedule: list of steps, a step = list of (request id, number of tokens).  Every position's
    logits are asked for; returns {id: [T, vocab] fp32}.  Requests end when their tokens do."""
    at = {k: 0 for k in toks}
    rows = {k: [] for k in toks}
    for step in schedule:
        entries, end, order = [], [], []
        for rid, n in step:
            lo = at[rid]
            entries.append((rid, toks[rid][lo:lo + n], list(range(n))))
            order += [rid] * n
            at[rid] = lo + n
            if at[rid] == len(toks[rid]):
                end.append(rid)
        out = eng.replay_step(entries, end)
        assert out.shape[0] == len(order)
        for j, rid in enumerate(order):
            rows[rid].append(out[j])
    assert all(at[k] == len(toks[k]) for k in toks), "schedule does not cover every token"
    return {k: torch.stack(v) for k, v in rows.items()}


def assert_matches_oracle(eng, cfg, weights, toks: dict, schedule, tol, oracle_cache=None):
    got = replay(eng, toks, schedule)
    worst = 0.0
    for rid, t in toks.items():
        key = tuple(t)
        if oracle_cache is not None and key in oracle_cache:
            want = oracle_cache[key]
        else:
            want = zo.forward(cfg, weights, t)
            if oracle_cache is not None:
                oracle_cache[key] = want
        err = zo.logit_error(got[rid], want)
        worst = max(worst, err)
        assert err < tol, f"request {rid} ({len(t)} tokens): logits differ from the oracle by {err:.3g} (limit {tol})"
    return worst


def portions(n, sizes):
    """Cut n tokens into portions cycling through ``sizes``."""
    out, i = [], 0
    while n > 0:
        k = min(n, sizes[i % len(sizes)])
        out.append(k)
        n -= k
        i += 1
    return out


def whole_schedule(toks):
    return [[(rid, len(t))] for rid, t in toks.items()]


def decode_schedule(toks, tail):
    s = []
    for rid, t in toks.items():
        head = max(1, len(t) - tail)
        s.append([(rid, head)])
        s += [[(rid, 1)] for _ in range(len(t) - head)]
    return s


def chunked_schedule(toks, sizes):
    s = []
    for rid, t in toks.items():
        s += [[(rid, k)] for k in portions(len(t), sizes)]
    return s


def mixed_schedule(toks, sizes, live=4, seed=3):
    """Up to ``live`` requests at a time, each step a random subset of them with portions of
    changing size beside single tokens; finished requests make room for the next ones, so state
    slots and pages are handed on."""
    g = random.Random(seed)
    waiting = list(toks)
    at = {k: 0 for k in toks}
    running, s = [], []
    while waiting or running:
        while waiting and len(running) < live:
            running.append(waiting.pop(0))
        step = []
        for rid in list(running):
            if len(running) > 1 and g.random() < 0.25:
                continue
            left = len(toks[rid]) - at[rid]
            n = min(left, g.choice(sizes))
            step.append((rid, n))
            at[rid] += n
            if at[rid] == len(toks[rid]):
                running.remove(rid)
        if step:
            s.append(step)
    return s


def greedy_reference(cfg, weights, prompt, n):
    """n greedy tokens from the oracle; also the smallest top-1 / top-2 logit gap met on the way."""
    t, gap = list(prompt), float("inf")
    for _ in range(n):
        lg = zo.forward(cfg, weights, t)[-1]
        top = torch.topk(lg, 2).values
        gap = min(gap, float(top[0] - top[1]))
        t.append(int(lg.argmax()))
    return t[len(prompt):], gap


def greedy_engine(eng, prompt_list, n):
    reqs = eng.generate(prompt_list, SamplingParams(max_new_tokens=n, temperature=0.0, ignore_eos=True))
    return [r.output_ids for r in reqs]


# ------------------------------------------------------------------------------ one mixer alone
F64 = torch.float64


def run_chunks(block, h, cuts, kv=None, page=16):
    """One sequence through ``block`` in portions ``cuts`` (state slot 1, a scattered page table)."""
    T = h.shape[0]
    n_pages = -(-T // page)
    table = torch.tensor([[7 + 2 * i for i in range(n_pages)]], dtype=torch.int32, device=h.device)
    block.alloc_state(3)
    outs, a = [], 0
    for n in cuts:
        pos = torch.arange(a, a + n, dtype=torch.int32, device=h.device)
        slots = (table[0, (pos // page).long()] * page + pos % page).to(torch.int32)
        meta = AttnMeta("prefill", pos, slots, table, cu_q=torch.tensor([0, n], dtype=torch.int32, device=h.device),
                        kv_lens=torch.tensor([a + n], dtype=torch.int32, device=h.device),
                        items=torch.tensor([[0, r] for r in range(0, n, 32)], dtype=torch.int32, device=h.device))
        seqs = (torch.tensor([0, n], dtype=torch.int32, device=h.device),
                torch.tensor([1], dtype=torch.int32, device=h.device),
                torch.tensor([int(a == 0)], dtype=torch.int32, device=h.device))
        outs.append(block.forward(h[a:a + n].contiguous(), MixerCtx(meta, kv, seqs)))
        a += n
    return torch.cat(outs)



def attention_block(a, width, dev, dt, max_pos=128):
    blk = GatedWindowAttention(0, width, a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["mask"]["size"],
                               a["mask"]["keep_first"], a["rot"]["base"], a["rot"]["dims"], a["scale"], 1e-5, max_pos,
                               dev, dt)
    return blk, PagedKVCache(1, 64, a["kv_heads"], blk.D, 16, dt, dev)


def _planted(dev, dt, tol, L, w, h, i, cuts, other_mask):
    a = L["mixer"]["left"]
    w64 = {k: v.to(F64) for k, v in w.items()}
    hq = h.to(dt).to(F64)                      # the oracle sees the inputs the block sees
    want = zo.window_attention(hq, w64, a, 1e-5)
    blk, kv = attention_block(a, h.shape[1], dev, dt)
    blk.load(w)
    got = run_chunks(blk, h.to(device=dev, dtype=dt), cuts, kv).cpu()
    rel = ((got.to(F64) - want).abs().max() / want.abs().max()).item()
    assert rel < tol, rel
    # the planted key matters: with the edge one token further / nearer the oracle's answer moves
    moved = zo.window_attention(hq, w64, dict(a, mask=other_mask), 1e-5)
    assert (moved[i] - want[i]).abs().max() > 0.08 * want[i].abs().max()


def planted_window_case(dev, dt, tol, gap, seen, cuts):
    """A key made to dominate the softmax whenever it is visible: the query's own input row,
    doubled (the projection-wide norm gives it the same key, its value is twice as large), sits
    ``gap`` tokens back (window 9: gap 8 is the last key inside, gap 9 the first outside); k uses
    q's weights, the scale is sharp and nothing is rotated, so one token off changes the output."""
    L = zo.parallel_layer(heads=2, kv_heads=2, dim=16, vdim=16, window=9, keep_first=0, rot_dims=0)
    L["mixer"]["left"]["scale"] = 6.0
    w = zo.sub(zo.random_weights(zo.make_config([L], width=24), 6), "l0.mix.left.")
    w["k"], w["k.norm"] = w["q"].clone(), w["q.norm"].clone()
    h = torch.randn(60, 24, generator=torch.Generator().manual_seed(4))
    h[59 - gap] = 2 * h[59]
    _planted(dev, dt, tol, L, w, h, 59, cuts, {"size": 8 if seen else 10, "keep_first": 0})


def planted_kept_case(dev, dt, tol, j, seen, cuts):
    """The same planting at the edge of the kept first tokens (keep_first 3: key 2 stays visible
    far behind the window, key 3 does not)."""
    L = zo.parallel_layer(heads=2, kv_heads=1, dim=16, vdim=12, window=6, keep_first=3, rot_dims=0)
    L["mixer"]["left"]["scale"] = 6.0
    w = zo.sub(zo.random_weights(zo.make_config([L], width=24), 7), "l0.mix.left.")
    w["k"], w["k.norm"] = w["q"][:16].clone(), w["q.norm"][:16].clone()
    h = torch.randn(50, 24, generator=torch.Generator().manual_seed(5))
    h[j] = 2 * h[49]
    _planted(dev, dt, tol, L, w, h, 49, cuts, {"size": 6, "keep_first": 2 if seen else 4})
