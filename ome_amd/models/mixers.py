"""Token mixers and feed-forwards as parameterised building blocks (every size and constant is a
constructor argument), for decoders that assemble their layers from a per-layer list.

* :class:`GatedWindowAttention` -- grouped-query attention over the paged KV cache with a sliding
  window that keeps the sequence's first tokens visible, projection-wide q / k RMSNorm, partial
  rotary embedding (interleaved or half-split pairs) and a sigmoid output gate;
* :class:`GatedDeltaMixer` -- the gated delta rule (short causal convolutions, unit-norm q / k,
  per-head decay and write strength, fp32 state per request slot);
* :class:`Mamba2Mixer` -- Mamba-2 / SSD selective scan with grouped B / C and a gated group norm;
* :class:`ClampedGLU` -- gated feed-forward ``min(g, L) * sigmoid(1.702 min(g, L)) * (clamp(u, -L, L) + 1)``.

Each block owns its weights (fused input projection, checkpoint tensors concatenated at load), its
recurrent state (``alloc_state``) and one ``forward(h, ctx)`` over a varlen batch of rows: prompt
chunks and single decode rows alike, described by :class:`MixerCtx`.  The projections run on the
framework's GEMM dispatch (``quant.linear``); everything between them is one of the HIP ops of
``ome_amd.ops`` (CPU tensors: their fp32 references).
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch

from ome_amd import ops
from ome_amd.models.common import AttnMeta, PagedKVCache, mixed_attention
from ome_amd.models.config import attn_tile_dim, plain_rope_table
from ome_amd.models.quant import linear


@dataclass
class MixerCtx:
    """One step's batch as the mixers see it: attention metadata + paged cache for the layers that
    own KV pages, ``seqs`` = (cu, slot, reset) row ranges / state slots / fresh-start flags for the
    recurrent ones."""
    meta: AttnMeta
    kv: PagedKVCache
    seqs: tuple


def paged_attention(q: torch.Tensor, k_cache, v_cache, meta: AttnMeta, scale: float, window: int = -1,
                    keep_first: int = 0) -> torch.Tensor:
    """Decode / prefill / mixed dispatch over the paged cache (q [T, Hq, D] -> [T, Hq, D])."""
    kw = dict(window=window, keep_first=keep_first)
    if meta.is_decode:
        return ops.paged_decode(q, k_cache, v_cache, meta.block_tables, meta.seq_lens, scale, meta.decode_ws,
                                order=meta.order, **kw)
    if meta.mode == "mixed":
        return mixed_attention(
            q, meta.num_prefill,
            lambda qp, op: ops.paged_prefill(qp, k_cache, v_cache, meta.block_tables, meta.cu_q, meta.kv_lens,
                                             meta.items, scale, out=op, **kw),
            lambda qd, od: ops.paged_decode(qd, k_cache, v_cache, meta.dec_block_tables, meta.seq_lens, scale,
                                            meta.decode_ws, out=od, order=meta.order, **kw))
    return ops.paged_prefill(q, k_cache, v_cache, meta.block_tables, meta.cu_q, meta.kv_lens, meta.items, scale,
                             **kw)


class _Block:
    """Weights as plain tensors; ``tensors()`` lists them for the byte count."""

    def __init__(self, device, dtype):
        self.device, self.dtype = torch.device(device), dtype

    def _put(self, t: torch.Tensor, dtype=None) -> torch.Tensor:
        return t.to(device=self.device, dtype=dtype or self.dtype).contiguous()

    def _rand(self, gen, *shape, std: float) -> torch.Tensor:
        return torch.empty(*shape, dtype=self.dtype, device=self.device).normal_(0.0, std, generator=gen)

    def tensors(self) -> list[torch.Tensor]:
        return [v for v in vars(self).values() if isinstance(v, torch.Tensor)]

    def alloc_state(self, slots: int) -> None:
        pass


class GatedWindowAttention(_Block):
    """q = W_q h, k = W_k h, v = W_v h; q and k each RMS-normalised over the WHOLE projection
    (all heads at once, weights of that width); rotary on the first ``rot_dims`` dims of every
    head; score = q.k * ``scale``; query i sees key j <= i when i - j < ``window`` or
    j < ``keep_first``; softmax; heads * sigmoid(W_g h); W_o.  Checkpoint tensors ``q k v q.norm
    k.norm g o``."""

    def __init__(self, layer: int, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                 keep_first: int, rot_base: float, rot_dims: int, scale: float, eps: float, max_positions: int,
                 device, dtype, interleaved: bool = True):
        super().__init__(device, dtype)
        if heads % kv_heads or heads // kv_heads > 16:
            raise ValueError(f"attention: {heads} query heads over {kv_heads} kv heads (groups of <= 16 supported)")
        self.layer, self.width, self.Hq, self.Hkv, self.dim, self.vdim = layer, width, heads, kv_heads, dim, vdim
        self.window, self.keep_first = int(window) if window and window > 0 else -1, int(keep_first)
        self.rot_dims, self.scale, self.eps, self.interleaved = int(rot_dims), float(scale), float(eps), interleaved
        self.D = attn_tile_dim(max(dim, vdim))
        self.cos_sin = plain_rope_table(rot_base, self.rot_dims, max_positions, self.device) if rot_dims else \
            torch.zeros(max_positions, 0, device=self.device)
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.w_in = self.qn = self.kn = self.w_o = None

    def load(self, t: dict) -> None:
        self.w_in = self._put(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0))
        self.qn, self.kn = self._put(t["q.norm"]), self._put(t["k.norm"])
        self.w_o = self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        self.w_in = self._rand(gen, self.nq + self.nk + self.nv + self.Hq * self.vdim, self.width, std=std)
        self.qn = torch.ones(self.nq, dtype=self.dtype, device=self.device)
        self.kn = torch.ones(self.nk, dtype=self.dtype, device=self.device)
        self.w_o = self._rand(gen, self.width, self.Hq * self.vdim, std=std)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        T = h.shape[0]
        nq, nk, nv = self.nq, self.nk, self.nv
        p = linear(h, self.w_in)                                   # [T, q | k | v | gate]
        q = torch.empty(T, self.Hq, self.D, dtype=h.dtype, device=h.device)
        k_cache, v_cache = ctx.kv.layer(self.layer)
        ops.wide_norm_rope_cache(p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:nq + nk + nv], ctx.meta.positions,
                                 self.cos_sin, self.rot_dims, self.interleaved, self.qn, self.kn, self.eps, q,
                                 k_cache, v_cache, ctx.meta.slots, self.Hq, self.Hkv, self.dim, self.vdim)
        a = paged_attention(q, k_cache, v_cache, ctx.meta, self.scale, self.window, self.keep_first)
        return linear(ops.head_gate(a, p[:, nq + nk + nv:], self.vdim, 0), self.w_o)


class GatedDeltaMixer(_Block):
    """Gated delta rule.  q, k (``kv_heads`` x ``dim``) and v (``heads`` x ``vdim``) pass a causal
    depthwise convolution of ``conv`` taps + SiLU; q, k become unit vectors per head (q also times
    dim^-1/2); per head, with g = exp(-exp(A_log) softplus(W_a h + dt_bias)), beta = sigmoid(W_b h):
    S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q.  Output: RMSNorm of each head's
    o times a shared weight times silu(W_g h), then W_o.  Checkpoint tensors ``q q.conv k k.conv v
    v.conv b a A_log dt_bias norm g o``; state: conv tail [slots, C, taps-1], S^T [slots, heads,
    vdim, dim] fp32."""

    def __init__(self, width: int, heads: int, kv_heads: int, dim: int, vdim: int, conv: int, eps: float, device,
                 dtype):
        super().__init__(device, dtype)
        if heads % kv_heads:
            raise ValueError(f"gated delta rule: {heads} value heads over {kv_heads} key heads")
        self.width, self.Hv, self.Hk, self.dk, self.dv, self.K, self.eps = width, heads, kv_heads, dim, vdim, conv, eps
        self.kd, self.vd = kv_heads * dim, heads * vdim
        self.cd = 2 * self.kd + self.vd
        self.w_in = self.conv_w = self.A_log = self.dt_bias = self.gnorm = self.w_o = None
        self.conv_state = self.rec_state = None

    def load(self, t: dict) -> None:
        self.w_in = self._put(torch.cat([t["q"], t["k"], t["v"], t["g"], t["b"], t["a"]], 0))
        self.conv_w = self._put(torch.cat([t["q.conv"], t["k.conv"], t["v.conv"]], 0))
        self.A_log, self.dt_bias = self._put(t["A_log"], torch.float32), self._put(t["dt_bias"], torch.float32)
        self.gnorm, self.w_o = self._put(t["norm"]), self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        f32 = dict(dtype=torch.float32, device=self.device)
        self.w_in = self._rand(gen, self.cd + self.vd + 2 * self.Hv, self.width, std=std)
        self.conv_w = self._rand(gen, self.cd, self.K, std=0.3)
        self.A_log = torch.log(torch.linspace(0.5, 8.0, self.Hv, **f32))
        self.dt_bias = torch.linspace(-1.0, 1.0, self.Hv, **f32)
        self.gnorm = torch.ones(self.dv, dtype=self.dtype, device=self.device)
        self.w_o = self._rand(gen, self.width, self.vd, std=std)

    def alloc_state(self, slots: int) -> None:
        self.conv_state = torch.zeros(slots, self.cd, max(self.K - 1, 0), dtype=self.dtype, device=self.device)
        self.rec_state = torch.zeros(slots, self.Hv, self.dv, self.dk, dtype=torch.float32, device=self.device)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        cu, slot, reset = ctx.seqs
        kd, vd, cd, Hv = self.kd, self.vd, self.cd, self.Hv
        p = linear(h, self.w_in)                                   # [T, q | k | v | gate | b | a]
        c = ops.ssm_conv1d(p[:, :cd], self.conv_w, None, self.conv_state, cu, slot, reset)
        o = ops.gdn_scan(c[:, :kd], c[:, kd:2 * kd], c[:, 2 * kd:], p[:, cd + vd + Hv:], p[:, cd + vd:cd + vd + Hv],
                         self.A_log, self.dt_bias, self.rec_state, cu, slot, reset, Hv, self.Hk)
        o = ops.gated_rmsnorm(o, p[:, cd:cd + vd], self.gnorm, self.dv, self.eps, norm_first=True, exact=True)
        return linear(o, self.w_o)


class Mamba2Mixer(_Block):
    """Mamba-2.  W_in h = [z | x | B | C | dt] (inner = heads * vdim, B / C ``groups`` x ``state``);
    x, B, C pass a causal depthwise convolution (``conv`` taps, bias) + SiLU; dt = softplus(dt +
    dt_bias); per head S <- exp(-exp(A_log) dt) S + dt B x^T, y = S^T C + D x; y * silu(z) is
    RMS-normalised in ``norm_groups`` equal parts, scaled, then W_o.  Checkpoint tensors ``in conv
    conv.b dt_bias A_log D norm o``; state: conv tail [slots, C, taps-1], S [slots, heads, vdim,
    state] fp32."""

    def __init__(self, width: int, heads: int, vdim: int, state: int, groups: int, conv: int, norm_groups: int,
                 eps: float, device, dtype):
        super().__init__(device, dtype)
        self.width, self.H, self.P, self.N, self.G, self.K, self.eps = width, heads, vdim, state, groups, conv, eps
        self.I = heads * vdim
        if heads % groups or self.I % norm_groups:
            raise ValueError(f"mamba2: {heads} heads / {groups} groups / {norm_groups} norm groups do not divide")
        self.cd = self.I + 2 * groups * state
        self.norm_group = self.I // norm_groups
        self.w_in = self.conv_w = self.conv_b = self.A = self.Dp = self.dt_bias = self.gnorm = self.w_o = None
        self.conv_state = self.ssm_state = None

    def load(self, t: dict) -> None:
        self.w_in, self.conv_w, self.conv_b = self._put(t["in"]), self._put(t["conv"]), self._put(t["conv.b"])
        self.A = -torch.exp(t["A_log"].float()).to(self.device)
        self.Dp, self.dt_bias = self._put(t["D"], torch.float32), self._put(t["dt_bias"], torch.float32)
        self.gnorm, self.w_o = self._put(t["norm"]), self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        f32 = dict(dtype=torch.float32, device=self.device)
        self.w_in = self._rand(gen, self.I + self.cd + self.H, self.width, std=std)
        self.conv_w, self.conv_b = self._rand(gen, self.cd, self.K, std=0.3), self._rand(gen, self.cd, std=std)
        self.A = -torch.linspace(0.5, 8.0, self.H, **f32)
        self.Dp = torch.ones(self.H, **f32)
        self.dt_bias = torch.full((self.H,), math.log(math.expm1(0.05)), **f32)
        self.gnorm = torch.ones(self.I, dtype=self.dtype, device=self.device)
        self.w_o = self._rand(gen, self.width, self.I, std=std)

    def alloc_state(self, slots: int) -> None:
        self.conv_state = torch.zeros(slots, self.cd, max(self.K - 1, 0), dtype=self.dtype, device=self.device)
        self.ssm_state = torch.zeros(slots, self.H, self.P, self.N, dtype=torch.float32, device=self.device)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        cu, slot, reset = ctx.seqs
        I, cd, GN = self.I, self.cd, self.G * self.N
        p = linear(h, self.w_in)                                   # [T, z | x B C | dt]
        c = ops.ssm_conv1d(p[:, I:I + cd], self.conv_w, self.conv_b, self.conv_state, cu, slot, reset)
        y = ops.ssm_scan(c[:, :I], p[:, I + cd:], c[:, I:I + GN], c[:, I + GN:], self.A, self.Dp, self.dt_bias, 0.0,
                         self.ssm_state, cu, slot, reset, self.H, self.P, self.N, self.G)
        y = ops.gated_rmsnorm(y, p[:, :I], self.gnorm, self.norm_group, self.eps, exact=True)
        return linear(y, self.w_o)


class ClampedGLU(_Block):
    """g = min(W_gate h, L), u = clamp(W_up h, -L, L); W_down (g sigmoid(1.702 g) (u + 1)).
    Checkpoint tensors ``gate up down``."""

    def __init__(self, width: int, ff: int, limit: float, device, dtype):
        super().__init__(device, dtype)
        self.width, self.ff, self.limit = width, ff, float(limit)
        self.w_gu = self.w_d = None

    def load(self, t: dict) -> None:
        self.w_gu, self.w_d = self._put(torch.cat([t["gate"], t["up"]], 0)), self._put(t["down"])

    def init_random(self, gen, std: float) -> None:
        self.w_gu, self.w_d = self._rand(gen, 2 * self.ff, self.width, std=std), self._rand(gen, self.width, self.ff,
                                                                                          std=std)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return linear(ops.act_and_mul(linear(h, self.w_gu), 2, limit=self.limit), self.w_d)
