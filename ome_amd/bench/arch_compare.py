"""Zavilorn beside the closest existing hybrid (NemotronH: Mamba-2 + attention + dense MLP) at equal
width, depth and mixer sizes, random weights: engine-level prefill / decode throughput, and a
per-kernel table that sets every kernel added for the design next to the like kernel of the
existing models with its share of the HBM roofline (``bench.py --arch-compare``).

Sizes resemble real layers (width 2048 / 4096, 128-wide heads, Mamba-2 heads of 64 x 128 state).
The Zavilorn stack is [parallel + feed-forward, mamba2, mamba2, mamba2] x 2; the NemotronH stack
``*-MMM*-MMM`` has the same attention, MLP width and Mamba-2 layers (it has no delta-rule mixer,
so its attention blocks are lighter; Qwen3-Next's Gated DeltaNet kernel is the delta rule's like
kernel in the table).
"""
from __future__ import annotations

import json
import time

import torch

HBM_GBS = 8000.0    # MI355X HBM3E peak, GB/s (the roofline of every kernel in the table)

SIZES = {
    "2k": dict(width=2048, heads=16, kv=4, ff=5632, mheads=64, vocab=32768),
    "4k": dict(width=4096, heads=32, kv=8, ff=14336, mheads=128, vocab=32768),
}


def zavilorn_config(s: dict, window: int = 1024, keep_first: int = 8) -> dict:
    par = {"type": "parallel",
           "mixer": {"left": {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128,
                              "mask": {"size": window, "keep_first": keep_first},
                              "rot": {"base": 10000.0, "dims": 64}, "scale": 128 ** -0.5},
                     "right": {"heads": s["heads"], "kv_heads": s["heads"] // 2, "dim": 128, "vdim": 128, "conv": 4},
                     "left_scale": 0.5, "right_scale": 0.5},
           "mlp": {"kind": "dense", "ff": s["ff"], "limit": 7.0}}
    mam = {"type": "mamba2", "mixer": {"heads": s["mheads"], "vdim": 64, "state": 128, "groups": 8, "conv": 4,
                                       "norm_groups": 8}, "mlp": None}
    return {"architecture": "Zavilorn", "embedding": {"scale": 1.0}, "layers": [par, mam, mam, mam] * 2,
            "norm": {"eps": 1e-6}, "vocab": s["vocab"], "width": s["width"], "max_positions": 8192}


def nemotron_config(s: dict) -> dict:
    return dict(architectures=["NemotronHForCausalLM"], model_type="nemotron_h", hidden_size=s["width"],
                hybrid_override_pattern="*-MMM*-MMM", num_attention_heads=s["heads"], num_key_value_heads=s["kv"],
                head_dim=128, intermediate_size=s["ff"], mlp_hidden_act="relu2", mamba_num_heads=s["mheads"],
                mamba_head_dim=64, ssm_state_size=128, n_groups=8, conv_kernel=4, vocab_size=s["vocab"],
                layer_norm_epsilon=1e-6, max_position_embeddings=8192, time_step_min=0.001, tie_word_embeddings=True)


def _engine(name: str, cfg: dict, max_running: int, context: int):
    from ome_amd.models.config import PRESETS
    from ome_amd.runtime.engine import Engine, EngineArgs

    PRESETS[name] = cfg
    return Engine(EngineArgs(model=name, device="cuda", load_format="dummy", max_running_requests=max_running,
                             context_length=context, chunked_prefill_size=4096, max_total_tokens=max_running * context,
                             watchdog_timeout=0.0, cuda_graph_max_bs=max_running))


def throughput(name: str, cfg: dict, prefill_len: int = 2048, prefill_n: int = 8, decode_bs: int = 32,
               decode_ctx: int = 1024, decode_n: int = 64) -> dict:
    """Prefill tokens/s (``prefill_n`` prompts of ``prefill_len``, one new token each) and decode
    tokens/s (``decode_bs`` requests at ~``decode_ctx`` context, ``decode_n`` tokens each, timed
    from the last first token to the end) through the engine's scheduler and HIP-graph decode."""
    import random

    from ome_amd.runtime.request import SamplingParams

    eng = _engine(name, cfg, max(decode_bs, prefill_n), prefill_len + decode_ctx)
    g = random.Random(0)
    V = cfg.get("vocab") or cfg.get("vocab_size")

    def toks(n):
        return [g.randrange(V) for _ in range(n)]

    one = SamplingParams(max_new_tokens=1, temperature=0.0, ignore_eos=True)
    eng.generate([toks(prefill_len)], one)                       # warm-up (allocations, GEMM heuristics)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.generate([toks(prefill_len) for _ in range(prefill_n)], one)
    torch.cuda.synchronize()
    pre = prefill_n * prefill_len / (time.perf_counter() - t0)
    reqs = eng.generate([toks(decode_ctx) for _ in range(decode_bs)],
                        SamplingParams(max_new_tokens=decode_n + 1, temperature=0.0, ignore_eos=True))
    first = max(r.token_times[0] for r in reqs)
    last = max(r.token_times[-1] for r in reqs)
    dec = decode_bs * decode_n / max(last - first, 1e-9)
    out = {"model": name, "prefill_tok_s": round(pre), "decode_tok_s": round(dec),
           "weights_GiB": round(eng.runner.model.weight_bytes() / 2 ** 30, 2)}
    del eng
    torch.cuda.empty_cache()
    return out


def _time_us(fn, iters: int = 30) -> float:
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) * 1000.0 / iters


def kernel_table(T: int = 4096, B: int = 64, ctx: int = 4096, width: int = 4096) -> list[dict]:
    """(kernel of the design, like kernel of an existing model) pairs at prefill (``T`` rows) and
    decode (``B`` rows, ``ctx`` context) sizes: microseconds, bytes that must move, share of the
    HBM roofline, and how much further from it the new kernel is (``vs_like`` <= 2 is the bar)."""
    from ome_amd import ops
    from ome_amd.models.config import plain_rope_table

    dev, bf = "cuda", torch.bfloat16
    rows = []

    def pair(name, new, like, bytes_new, bytes_like, note=""):
        tn, tl = _time_us(new), _time_us(like)
        fn, fl = bytes_new / tn / 1e3 / HBM_GBS, bytes_like / tl / 1e3 / HBM_GBS
        rows.append({"kernel": name, "us": round(tn, 1), "roofline": round(fn, 3), "like_us": round(tl, 1),
                     "like_roofline": round(fl, 3), "vs_like": round(fl / max(fn, 1e-9), 2), "note": note})

    torch.manual_seed(0)
    for R, tag in ((T, "prefill"), (B, "decode")):
        # ---- residual add + RMSNorm: fp32 residual vs the bf16-residual kernel
        res = torch.randn(R, width, device=dev)
        x1 = torch.randn(R, width, device=dev).to(bf)
        x2 = torch.randn(R, width, device=dev).to(bf)
        w = torch.ones(width, device=dev, dtype=bf)
        rb, xb = res.to(bf), x1.clone()
        pair(f"residual_rmsnorm 1 addend ({tag})", lambda: ops.residual_rmsnorm(res, w, 1e-6, x1, 1.0),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 12, R * width * 8,
             "fp32 residual: 12 B / element against 8")
        pair(f"residual_rmsnorm 2 addends ({tag})", lambda: ops.residual_rmsnorm(res, w, 1e-6, x1, 0.5, x2, 0.5),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 14, R * width * 8)
        # ---- q/k norm + rotary + paged write
        Hq, Hkv, D, P = 32, 8, 128, 16
        n_pages = R // P + 2
        kc = torch.zeros(n_pages, Hkv, P, D, device=dev, dtype=bf)
        vc = torch.zeros(n_pages, Hkv, D, P, device=dev, dtype=bf)
        qkv = torch.randn(R, (Hq + 2 * Hkv) * D, device=dev).to(bf)
        pos = torch.arange(R, dtype=torch.int32, device=dev)
        slots = pos + P
        cs = plain_rope_table(10000.0, 64, R + 1, dev)
        qo = torch.empty(R, Hq, D, device=dev, dtype=bf)
        qn, kn = torch.ones(Hq * D, device=dev, dtype=bf), torch.ones(Hkv * D, device=dev, dtype=bf)
        hn = torch.ones(D, device=dev, dtype=bf)
        nb = R * (Hq + 2 * Hkv) * D * 2 * 2
        pair(f"wide_norm_rope_cache ({tag})",
             lambda: ops.wide_norm_rope_cache(qkv[:, :Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D:],
                                              pos, cs, 64, True, qn, kn, 1e-6, qo, kc, vc, slots, Hq, Hkv, D, D),
             lambda: ops.rope_qkv_cache(qkv, pos, cs, 64, qo, kc, vc, slots, Hq, Hkv, D, True, hn, hn, 1e-6), nb, nb,
             "projection-wide norm: two passes over q / k")
        # ---- output gate
        o = torch.randn(R, Hq, D, device=dev).to(bf)
        gt = torch.randn(R, Hq * D, device=dev).to(bf)
        pair(f"head_gate ({tag})", lambda: ops.head_gate(o, gt, D, 0),
             lambda: o.view(R, Hq * D) * torch.sigmoid(gt), R * Hq * D * 6, R * Hq * D * 8,
             "like: the two eager elementwise kernels of the gated attention of Qwen3-Next")
        # ---- clamped GLU (same kernel, runtime limit)
        I = 14336
        gu = torch.randn(R, 2 * I, device=dev).to(bf)
        pair(f"act_and_mul limit ({tag})", lambda: ops.act_and_mul(gu, 2, limit=3.0), lambda: ops.act_and_mul(gu, 2),
             R * I * 6, R * I * 6)
    # ---- attention: decode over a long context, window + kept first keys vs the plain window
    Hq, Hkv, D, P, W = 32, 8, 128, 16, 1024
    per = ctx // P
    kc = (torch.randn(B * per + 1, Hkv, P, D, device=dev) * 0.3).to(bf)
    vc = (torch.randn(B * per + 1, Hkv, D, P, device=dev) * 0.3).to(bf)
    bt = (torch.arange(B * per, dtype=torch.int32, device=dev) + 1).view(B, per)
    sl = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q = torch.randn(B, Hq, D, device=dev).to(bf)
    ws = ops.DecodeWorkspace(B, Hq, D, ctx, 0, dev, parts=4)
    kvb = B * Hkv * D * 2 * 2
    pair("paged_decode window 1024 + 8 kept", lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W, keep_first=8),
         lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W), kvb * (W + 32), kvb * W,
         "one more 32-key tile per sequence for the kept keys")
    # ---- attention: prefill, 2 x 2048 rows
    q_lens = [2048, 2048]
    Tq = sum(q_lens)
    qp = torch.randn(Tq, Hq, D, device=dev).to(bf)
    cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
    kl = torch.tensor(q_lens, dtype=torch.int32, device=dev)
    bt2 = (torch.arange(2 * 128, dtype=torch.int32, device=dev) + 1).view(2, 128)
    items = torch.tensor(ops.prefill_work_items(q_lens, q_lens), dtype=torch.int32, device=dev)
    flops = 4.0 * Hq * D * sum(min(W + 8, i + 1) for i in range(2048)) * 2
    tn = _time_us(lambda: ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W, keep_first=8))
    tl = _time_us(lambda: ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W))
    rows.append({"kernel": "paged_prefill window 1024 + 8 kept (2 x 2048 rows)", "us": round(tn, 1),
                 "roofline": round(flops / tn / 1e6 / 2.5e3, 3), "like_us": round(tl, 1),
                 "like_roofline": round(flops / tl / 1e6 / 2.5e3, 3), "vs_like": round(tn / tl, 2),
                 "note": "share of 2.5 PFLOP/s bf16; like: the 4-wave GQA-4 kernel with a plain window"})
    return rows


def run(sizes=("2k", "4k"), kernels: bool = True, only: str | None = None) -> dict:
    out = {"throughput": [], "kernels": []}
    for k in sizes:
        s = SIZES[k]
        if only in (None, "zavilorn"):
            out["throughput"].append(throughput(f"zavilorn-{k}", zavilorn_config(s)))
        if only in (None, "nemotron"):
            out["throughput"].append(throughput(f"nemotron-h-like-{k}", nemotron_config(s)))
    if kernels:
        out["kernels"] = kernel_table()
    return out


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--sizes", default="2k,4k")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--only", choices=["zavilorn", "nemotron"], default=None, help="one stack (for kernel traces)")
    a = ap.parse_args(argv)
    res = run(tuple(a.sizes.split(",")), not a.no_kernels, a.only)
    for r in res["throughput"]:
        print(json.dumps(r))
    for r in res["kernels"]:
        print(json.dumps(r))
    return 0


if __name__ == "__main__":   # (run as a file under a profiler: make the package importable)
    import os
    import sys

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
    sys.exit(main())
