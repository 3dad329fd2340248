"""Slow fp64 implementation of the Metitar design, one function per mechanism, written from the
equations alone (no code shared with ``ome_amd``), plus makers of small random configs and
checkpoints for the tests."""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


# ------------------------------------------------------------------------------------ pieces
def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def silu(x):
    return x / (1 + torch.exp(-x))


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(h, w):
    """y_t = sum_j w[:, j] h_{t - K + 1 + j}, rows before the start are zero; h [T, C], w [C, K]."""
    T, K = h.shape[0], w.shape[1]
    y = torch.zeros_like(h)
    for t in range(T):
        for j in range(K):
            s = t - K + 1 + j
            if s >= 0:
                y[t] += w[:, j] * h[s]
    return y


def rotary_angles(rot, positions):
    """(cos, sin) [T, dims/2] with YaRN frequency scaling and amplitude factor."""
    dims, base = rot["dims"], float(rot["base"])
    amp = 1.0
    freq = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            def dim_of(turns):
                return dims * math.log(sc["original"] / (2 * math.pi * turns)) / (2 * math.log(base))
            lo = max(math.floor(dim_of(sc["fast"])), 0)
            hi = min(math.ceil(dim_of(sc["slow"])), dims - 1)
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f = f / sc["factor"] * ramp + f * (1 - ramp)
        freq.append(f)
    if sc:
        amp = 0.1 * math.log(sc["factor"]) + 1.0
    ang = torch.tensor(positions, dtype=F64)[:, None] * torch.tensor(freq, dtype=F64)[None]
    return torch.cos(ang) * amp, torch.sin(ang) * amp


def rotate_half(x, cos, sin):
    """x [T, dims] or [T, H, dims]: dim i pairs with i + dims/2."""
    half = x.shape[-1] // 2
    u, v = x[..., :half], x[..., half:]
    if x.dim() == 3:
        cos, sin = cos[:, None], sin[:, None]
    return torch.cat([u * cos - v * sin, v * cos + u * sin], -1)


def latent_kv(h, w, m, eps):
    """(latent c [T, kv_rank], rotated shared key [T, rot_dim]) of a layer that owns W_dkv."""
    R = m["kv_rank"]
    kv = h @ w["dkv"].T
    cos, sin = rotary_angles(m["rot"], list(range(h.shape[0])))
    return rms_unit(kv[:, :R], eps) * w["dkv.norm"], rotate_half(kv[:, R:], cos, sin)


def latent_attention(h, w, m, eps, kv=None, hide=None):
    """h [T, W] -> [T, W].  ``kv``: another layer's (c, rotated key) when this layer has none of its
    own.  ``hide`` = (i, j): query i does not see key j (to show that a key matters)."""
    T, H, d, r, vd = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = kv if kv is not None else latent_kv(h, w, m, eps)
    cq = rms_unit(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(T, H, d + r)
    cos, sin = rotary_angles(m["rot"], list(range(T)))
    qn, qr = q[..., :d], rotate_half(q[..., d:], cos, sin)
    kn = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, vd)
    out = torch.zeros(T, H, vd, dtype=F64)
    for hd in range(H):
        sink = float(w["sink"][hd])
        for i in range(T):
            s = (kn[:i + 1, hd] @ qn[i, hd] + kr[:i + 1] @ qr[i, hd]) * m["scale"]
            if hide is not None and hide[0] == i:
                s[hide[1]] = -math.inf
            top = max(float(s.max()), sink)
            e = torch.exp(s - top)
            out[i, hd] = (e / (e.sum() + math.exp(sink - top))) @ v[:i + 1, hd]
    return out.reshape(T, H * vd) @ w["o"].T


def hgrn2(h, w, m, eps):
    T, H, d, vd = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w["q"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, vd)
    low = w["lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ w["f"].T + w["f.b"])).view(T, H, d)
    S = torch.zeros(H, d, vd, dtype=F64)
    out = torch.zeros(T, H, vd, dtype=F64)
    for t in range(T):
        for hd in range(H):
            S[hd] = f[t, hd][:, None] * S[hd] + torch.outer(1 - f[t, hd], v[t, hd])
            out[t, hd] = S[hd].T @ q[t, hd]
    out = rms_unit(out, eps) * w["norm"]
    return out.reshape(T, H * vd) @ w["o"].T


def polynorm_ff(x, w, eps):
    z = x @ w["up"].T
    a, b, c, e = (float(t) for t in w["act"])
    return (a * rms_unit(z, eps) + b * rms_unit(z * z, eps) + c * rms_unit(z * z * z, eps) + e) @ w["down"].T


def swiglu(x, w, pre):
    return (silu(x @ w[pre + "gate"].T) * (x @ w[pre + "up"].T)) @ w[pre + "down"].T


def moe_ff(x, w, f):
    s = torch.sigmoid(x @ w["router"].T)
    y = torch.zeros_like(x)
    for t in range(x.shape[0]):
        for e in torch.topk(s[t], f["router"]["top"]).indices.tolist():
            y[t] += swiglu(s[t, e] * x[t], w, f"e{e}.")
    if f.get("shared"):
        y = y + swiglu(x, w, "shared.")
    return y


def router_margin(x, w, f):
    """Smallest gap between the last chosen and the first unchosen router score."""
    s = torch.sigmoid(x @ w["router"].T).sort(-1, descending=True).values
    k = f["router"]["top"]
    return float((s[:, k - 1] - s[:, k]).min()) if s.shape[1] > k else float("inf")


def side_input(x, tokens, table, w, layer, dim, eps):
    e = table[torch.tensor(tokens)][:, layer * dim:(layer + 1) * dim]
    y = (gelu_tanh(x @ w["gate"].T) * e) @ w["proj"].T
    return rms_unit(y, eps) * w["norm"]


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, residuals=None, margins=None):
    """Token ids -> fp64 logits [T, vocab]; ``residuals`` (a list) collects the stream after every
    layer, ``margins`` (a list) every routed layer's smallest router margin."""
    w = {k: v.to(F64) for k, v in weights.items() if v.is_floating_point()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    kv = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = x + causal_conv(x, w[p + "canon1"]) if cfg.get("canon") else x
        if L["type"] == "latent_attention":
            mw = sub(w, p + "mix.")
            if m.get("kv_from") is None:
                kv[i] = latent_kv(h, mw, m, eps)
            y = latent_attention(h, mw, m, eps, kv[i if m.get("kv_from") is None else m["kv_from"]])
        else:
            y = hgrn2(h, sub(w, p + "mix."), m, eps)
        x = x + layer_norm(y, w[p + "norm1"], w[p + "norm1.b"], eps)
        f = L.get("mlp")
        if f:
            y = polynorm_ff(x, sub(w, p + "mlp."), eps) if f["kind"] == "dense" else moe_ff(x, sub(w, p + "mlp."), f)
            if margins is not None and f["kind"] == "moe":
                margins.append(router_margin(x, sub(w, p + "mlp."), f))
            x = x + layer_norm(y, w[p + "norm2"], w[p + "norm2.b"], eps)
        if cfg.get("token_side"):
            x = x + side_input(x, tokens, w["side.embed"], sub(w, p + "side."), i, cfg["token_side"]["dim"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T * cfg.get("logit_scale", 1.0)


# ------------------------------------------------------------------------------------ makers
def attention_layer(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=12, q_rank=10, base=100.0, scaling="default",
                    scale=0.4, kv_from=None, mlp=None):
    if scaling == "default":
        scaling = {"factor": 4.0, "original": 16, "fast": 4.0, "slow": 1.0}
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank,
         "rot": rot, "scale": scale}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def hgrn2_layer(heads=2, dim=6, vdim=10, mlp=None):
    return {"type": "hgrn2", "mixer": {"heads": heads, "dim": dim, "vdim": vdim}, "mlp": mlp}


def dense(ff=40):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=12, shared=20):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


def make_config(layers, width=24, vocab=53, embed_scale=3.0, eps=1e-5, taps=3, side=4, logit_scale=1.5):
    cfg = {"architecture": "Metitar", "embedding": {"scale": embed_scale}, "layers": layers, "norm": {"eps": eps},
           "vocab": vocab, "width": width, "logit_scale": logit_scale}
    if taps:
        cfg["canon"] = {"taps": taps}
    if side:
        cfg["token_side"] = {"dim": side}
    return cfg


def random_weights(cfg, seed=0, gain=1.0):
    """bf16 tensors under the checkpoint's names; scales chosen so that every branch matters
    (``gain`` < 1 flattens every projection: a smoother model for 16-bit runs, whose rounding a
    stack of output norms otherwise amplifies)."""
    g = torch.Generator().manual_seed(seed)
    W, V, n = cfg["width"], cfg["vocab"], len(cfg["layers"])
    bf = torch.bfloat16

    def mat(o, i, s=1.0):
        return (torch.randn(o, i, generator=g) * s * gain / math.sqrt(i)).to(bf)

    def vec(k, lo, hi):
        return (torch.rand(k, generator=g) * (hi - lo) + lo).to(bf)

    t = {"embed": (torch.randn(V, W, generator=g) * 0.5).to(bf), "final.norm": vec(W, 0.7, 1.3),
         "final.norm.b": vec(W, -0.2, 0.2), "head": mat(V, W, 2.0)}
    if cfg.get("token_side"):
        t["side.embed"] = torch.randn(V, n * cfg["token_side"]["dim"], generator=g).to(bf)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"], t[p + "norm1.b"] = vec(W, 0.7, 1.3), vec(W, -0.2, 0.2)
        if cfg.get("canon"):
            t[p + "canon1"] = (torch.randn(W, cfg["canon"]["taps"], generator=g) * 0.4).to(bf)
        q = p + "mix."
        if L["type"] == "latent_attention":
            H, d, r, vd, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            t[q + "dq"], t[q + "dq.norm"], t[q + "uq"] = mat(Q, W, 2.0), vec(Q, 0.8, 1.6), mat(H * (d + r), Q, 3.0)
            if m.get("kv_from") is None:
                t[q + "dkv"], t[q + "dkv.norm"] = mat(R + r, W, 2.0), vec(R, 0.8, 1.6)
            t[q + "uk"], t[q + "uv"] = mat(H * d, R, 3.0), mat(H * vd, R, 2.0)
            t[q + "sink"], t[q + "o"] = vec(H, 0.5, 3.0), mat(W, H * vd, 2.0)
        else:
            H, d, vd = m["heads"], m["dim"], m["vdim"]
            t[q + "q"], t[q + "f"], t[q + "v"] = mat(H * d, W, 2.0), mat(H * d, W, 3.0), mat(H * vd, W, 2.0)
            t[q + "f.b"], t[q + "lower"] = vec(H * d, -1.0, 2.0), vec(H * d, 0.0, 0.9)
            t[q + "norm"], t[q + "o"] = vec(vd, 0.7, 1.3), mat(W, H * vd, 2.0)
        f = L.get("mlp")
        if f:
            t[p + "norm2"], t[p + "norm2.b"] = vec(W, 0.7, 1.3), vec(W, -0.2, 0.2)
            q = p + "mlp."
            if f["kind"] == "dense":
                t[q + "up"], t[q + "down"] = mat(f["ff"], W, 2.0), mat(W, f["ff"], 2.0)
                t[q + "act"] = torch.tensor([0.9, -0.5, 0.4, 0.1]).to(bf)
            else:
                t[q + "router"] = mat(f["router"]["experts"], W, 0.3 / gain)   # (scores off saturation; not flattened)
                names = [f"e{e}." for e in range(f["router"]["experts"])] + (["shared."] if f.get("shared") else [])
                for nm in names:
                    ff = f["shared"]["ff"] if nm == "shared." else f["expert"]["ff"]
                    t[q + nm + "gate"], t[q + nm + "up"], t[q + nm + "down"] = mat(ff, W, 2.0), mat(ff, W, 2.0), mat(W, ff, 2.0)
        if cfg.get("token_side"):
            q, sd = p + "side.", cfg["token_side"]["dim"]
            t[q + "gate"], t[q + "proj"], t[q + "norm"] = mat(sd, W, 2.0), mat(W, sd, 2.0), vec(W, 0.3, 0.9)
    return t


def save_model(folder, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return str(folder)


def logit_errors(got, want):
    """Per position: root mean square over the vocabulary of the centred difference, relative to the
    rms of the oracle's centred logits."""
    got, want = got.to(F64), want.to(F64)
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    ref = want - want.mean(-1, keepdim=True)
    return d.pow(2).mean(-1).sqrt() / ref.pow(2).mean().sqrt()


def logit_error(got, want):
    return logit_errors(got, want).max().item()
