"""Slow fp64 oracle of the Zavilorn design, written straight from its equations: one function per
mechanism, whole sequences at once, no cache, no batching, no code shared with ``ome_amd``.

Also the helpers the tests use to make small random models (config dict + tensors) and to save
them as a checkpoint folder.
"""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


# ------------------------------------------------------------------------------ mechanisms
def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def causal_conv_silu(x, w, b=None):
    """x [T, C]; w [C, taps], the LAST column multiplies the current token; zeros before t = 0."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                y[t] += w[:, j] * x[src]
    if b is not None:
        y = y + b
    return silu(y)


def rotate_pairs(x, base, dims, first_pos=0):
    """x [T, heads, d]: dims (2i, 2i+1), i < dims/2, turn by angle pos * base^(-2i/dims)."""
    T = x.shape[0]
    out = x.clone()
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        ang = (torch.arange(T, dtype=F64) + first_pos) * f
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(i, j, window, keep_first):
    return j <= i and (i - j < window or j < keep_first)


def window_attention(h, w, m, eps):
    """The left mixer of a parallel block."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rms_unit(h @ w["q"].T, eps) * w["q.norm"]          # one mean square over the whole projection
    k = rms_unit(h @ w["k"].T, eps) * w["k.norm"]
    v = (h @ w["v"].T).view(T, G, dv)
    q = rotate_pairs(q.view(T, H, d), m["rot"]["base"], m["rot"]["dims"])
    k = rotate_pairs(k.view(T, G, d), m["rot"]["base"], m["rot"]["dims"])
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        for i in range(T):
            js = [j for j in range(T) if visible(i, j, m["mask"]["size"], m["mask"]["keep_first"])]
            sc = torch.stack([(q[i, hh] * k[j, g]).sum() for j in js]) * m["scale"]
            p = torch.softmax(sc, 0)
            out[i, hh] = (p[:, None] * v[js, g]).sum(0)
    gate = torch.sigmoid(h @ w["g"].T)
    return (out.reshape(T, H * dv) * gate) @ w["o"].T


def gated_delta(h, w, m, eps):
    """The right mixer of a parallel block."""
    T = h.shape[0]
    H, Hk, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = causal_conv_silu(h @ w["q"].T, w["q.conv"]).view(T, Hk, d)
    k = causal_conv_silu(h @ w["k"].T, w["k.conv"]).view(T, Hk, d)
    v = causal_conv_silu(h @ w["v"].T, w["v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)
    decay = torch.exp(-torch.exp(w["A_log"]) * softplus(h @ w["a"].T + w["dt_bias"]))
    o = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        kh = hh // (H // Hk)
        S = torch.zeros(d, dv, dtype=F64)
        for t in range(T):
            S = decay[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hh] = S.T @ q[t, kh]
    o = rms_unit(o, eps) * w["norm"] * silu(h @ w["g"].T).view(T, H, dv)
    return o.reshape(T, H * dv) @ w["o"].T


def mamba2(h, w, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    z, x, B, C, dt = torch.split(h @ w["in"].T, [inner, inner, G * N, G * N, H], -1)
    xbc = causal_conv_silu(torch.cat([x, B, C], -1), w["conv"], w["conv.b"])
    x, B, C = torch.split(xbc, [inner, G * N, G * N], -1)
    x, B, C = x.reshape(T, H, P), B.reshape(T, G, N), C.reshape(T, G, N)
    dt = softplus(dt + w["dt_bias"])
    y = torch.zeros(T, H, P, dtype=F64)
    for hh in range(H):
        g = hh // (H // G)
        S = torch.zeros(N, P, dtype=F64)
        for t in range(T):
            S = torch.exp(-torch.exp(w["A_log"][hh]) * dt[t, hh]) * S + dt[t, hh] * torch.outer(B[t, g], x[t, hh])
            y[t, hh] = S.T @ C[t, g] + w["D"][hh] * x[t, hh]
    y = y.reshape(T, inner) * silu(z)                       # gate first, then the group norm
    ng = m["norm_groups"]
    y = rms_unit(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w["norm"]
    return y @ w["o"].T


def clamped_glu(h, w, f):
    lim = f["limit"]
    g = torch.clamp(h @ w["gate"].T, max=lim)
    u = torch.clamp(h @ w["up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w["down"].T


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, residuals=None):
    """tokens (list of int) -> fp64 logits [T, vocab]; ``residuals`` collects x after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = rms_unit(x, eps) * W[p + "norm1"]
        m = L["mixer"]
        if L["type"] == "mamba2":
            x = x + mamba2(h, sub(W, p + "mix."), m, eps)
        else:
            x = x + m["left_scale"] * window_attention(h, sub(W, p + "mix.left."), m["left"], eps) \
                + m["right_scale"] * gated_delta(h, sub(W, p + "mix.right."), m["right"], eps)
        if L["mlp"] is not None:
            x = x + clamped_glu(rms_unit(x, eps) * W[p + "norm2"], sub(W, p + "mlp."), L["mlp"])
        if residuals is not None:
            residuals.append(x.clone())
    return (rms_unit(x, eps) * W["final.norm"]) @ W["embed"].T


# ------------------------------------------------------------------------------ random models
def parallel_layer(heads=2, kv_heads=1, dim=24, vdim=16, window=9, keep_first=2, rot_dims=8, rot_base=100.0,
                   r_heads=2, r_kv_heads=1, r_dim=12, r_vdim=20, r_conv=3, ff=40, limit=1.25, left_scale=0.7,
                   right_scale=0.4):
    return {"type": "parallel",
            "mixer": {"left": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                               "mask": {"size": window, "keep_first": keep_first},
                               "rot": {"base": rot_base, "dims": rot_dims}, "scale": 1.3 / math.sqrt(dim)},
                      "right": {"heads": r_heads, "kv_heads": r_kv_heads, "dim": r_dim, "vdim": r_vdim,
                                "conv": r_conv},
                      "left_scale": left_scale, "right_scale": right_scale},
            "mlp": None if not ff else {"kind": "dense", "ff": ff, "limit": limit}}


def mamba_layer(heads=2, vdim=8, state=12, groups=1, conv=4, norm_groups=2, ff=0, limit=2.0):
    return {"type": "mamba2",
            "mixer": {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
                      "norm_groups": norm_groups},
            "mlp": None if not ff else {"kind": "dense", "ff": ff, "limit": limit}}


def make_config(layers, width=48, vocab=61, embed_scale=3.0, eps=1e-5):
    return {"architecture": "Zavilorn", "embedding": {"scale": embed_scale}, "layers": layers,
            "norm": {"eps": eps}, "vocab": vocab, "width": width}


def random_weights(cfg, seed=0, gain=1.0):
    """bf16 tensors under the checkpoint's names; scales chosen so every branch matters."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s * gain / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, lo, hi):
        return (torch.rand(n, generator=g) * (hi - lo) + lo).to(torch.bfloat16)

    t = {"embed": (torch.randn(cfg["vocab"], W, generator=g) * 0.5).to(torch.bfloat16), "final.norm": vec(W, 0.7, 1.3)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = vec(W, 0.7, 1.3)
        if L["type"] == "parallel":
            a, r = m["left"], m["right"]
            q = p + "mix.left."
            t[q + "q"], t[q + "k"] = mat(a["heads"] * a["dim"], W, 2.0), mat(a["kv_heads"] * a["dim"], W, 2.0)
            t[q + "v"], t[q + "g"] = mat(a["kv_heads"] * a["vdim"], W), mat(a["heads"] * a["vdim"], W)
            t[q + "q.norm"], t[q + "k.norm"] = vec(a["heads"] * a["dim"], 0.8, 2.0), vec(a["kv_heads"] * a["dim"], 0.8, 2.0)
            t[q + "o"] = mat(W, a["heads"] * a["vdim"], 2.0)
            q = p + "mix.right."
            kd, vd = r["kv_heads"] * r["dim"], r["heads"] * r["vdim"]
            t[q + "q"], t[q + "k"], t[q + "v"] = mat(kd, W, 2.0), mat(kd, W, 2.0), mat(vd, W, 2.0)
            for n, c in (("q", kd), ("k", kd), ("v", vd)):
                t[q + n + ".conv"] = (torch.randn(c, r["conv"], generator=g) * 0.6).to(torch.bfloat16)
            t[q + "b"], t[q + "a"] = mat(r["heads"], W, 2.0), mat(r["heads"], W, 2.0)
            t[q + "A_log"] = vec(r["heads"], -1.5, 0.5)
            t[q + "dt_bias"] = vec(r["heads"], -1.0, 1.0)
            t[q + "norm"] = vec(r["vdim"], 0.7, 1.3)
            t[q + "g"], t[q + "o"] = mat(vd, W, 2.0), mat(W, vd, 2.0)
        else:
            q = p + "mix."
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            t[q + "in"] = mat(2 * inner + 2 * gn + m["heads"], W, 2.0)
            t[q + "conv"] = (torch.randn(inner + 2 * gn, m["conv"], generator=g) * 0.6).to(torch.bfloat16)
            t[q + "conv.b"] = vec(inner + 2 * gn, -0.2, 0.2)
            t[q + "dt_bias"] = vec(m["heads"], -2.0, 0.5)
            t[q + "A_log"] = vec(m["heads"], -1.5, 1.0)
            t[q + "D"] = vec(m["heads"], 0.5, 1.5)
            t[q + "norm"] = vec(inner, 0.7, 1.3)
            t[q + "o"] = mat(W, inner, 2.0)
        if L["mlp"] is not None:
            t[p + "norm2"] = vec(W, 0.7, 1.3)
            q = p + "mlp."
            t[q + "gate"], t[q + "up"] = mat(L["mlp"]["ff"], W, 3.0), mat(L["mlp"]["ff"], W, 3.0)
            t[q + "down"] = mat(W, L["mlp"]["ff"], 2.0)
    return t


def save_model(folder, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)


def logit_error(got, want):
    """Root mean square over the vocabulary of the centred difference, relative to the rms of the
    oracle's centred logits."""
    got, want = got.to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return (d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()).max().item()
