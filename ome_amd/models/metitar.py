"""Metitar: a layer-list decoder (``architecture: Metitar``) with a post-norm fp32 residual stream.

``layers[i]`` = {``type``, ``mixer`` (that mixer's own sizes), ``mlp`` (or null)}.  Mixer types:

* ``latent_attention`` -- ``mixers.LatentAttention`` (``mixer.kv_from: j`` = no key/value projection
  of its own: it attends over layer j's cached latent and rotary key);
* ``hgrn2`` -- ``mixers.Hgrn2Mixer``.

Feed-forwards (``mlp.kind``): ``dense`` = ``mixers.PolyNormMLP``, ``moe`` = ``mixers.InputScaledMoE``.

One layer, with x the fp32 stream:

  h = x + causal_conv(x)              (``canon.taps`` taps per channel, ``l<i>.canon1``; absent: h = x)
  x += LayerNorm(mixer(h))            (``l<i>.norm1`` / ``.norm1.b``: the norm sits on the sublayer's OUTPUT)
  x += LayerNorm(ff(x))               (``l<i>.norm2`` / ``.norm2.b``; layers without an mlp skip this)
  x += RMSNorm(side_i(x, token)) w    (``mixers.TokenSideInput`` with ``side.embed``; ``token_side`` absent: skipped)

x starts as ``embed[token] * embedding.scale``; logits = ``head`` . LayerNorm(x)(``final.norm``) *
``logit_scale``.

Numerics: x is fp32 from the embedding to the final norm (``ops.embedding_f32``,
``ops.post_norm_add``, ``ops.conv_mix`` with an fp32 tail state); GEMMs run in the model dtype
with fp32 accumulation on the stream rounded once per sublayer; attention scores / softmax, every
norm, rotary angles, router logits, gates, the recurrence and its state are fp32 inside the
kernels; logits leave the head in fp32.

Cache and state: latent-attention layers that own a key/value projection own KV pages
(``kv_layers``; one shared row per token: in bf16 ``[latent | rotary key]`` padded to a shape of the
latent kernel, values read from the same row; in fp32 key rows + value columns of the generic
kernels); per request slot every
layer keeps its conv tail and every HGRN2 layer its fp32 state (``alloc_state``).  Prefix caching
is off (``stateful``).  The model has no cache, loop or scheduler of its own: ``ModelRunner``
drives it like the other hybrids.
"""
from __future__ import annotations

import torch

from ome_amd import ops
from ome_amd.models.common import AttnMeta, PagedKVCache
from ome_amd.models.config import ModelConfig
from ome_amd.models.llama import LlamaForCausalLM
from ome_amd.models.mixers import (Hgrn2Mixer, InputScaledMoE, LatentAttention, MixerCtx, PolyNormMLP,
                                   TokenSideInput)
from ome_amd.parallel import state as pstate

METITAR_ARCHS = {"Metitar"}


class MetitarForCausalLM(LlamaForCausalLM):
    stateful = True
    tune_gemms = False   # odd projection widths: the library heuristic, no TunableOp pass

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16, max_positions: int | None = None):
        st = pstate.get()
        if st.tp_size > 1 or st.pp_size > 1:
            raise NotImplementedError("Metitar: tensor / pipeline parallelism (one GPU holds the model)")
        super().__init__(cfg, device, dtype, 1)   # (the base's rotary table is unused: one row)
        hf = cfg.extra or {}
        W, eps = cfg.hidden_size, cfg.rms_norm_eps
        mp = max_positions or cfg.max_position_embeddings
        self.embed_scale = float((hf.get("embedding") or {}).get("scale", 1.0))
        self.logit_scale = float(hf.get("logit_scale", 1.0))
        self.taps = int((hf.get("canon") or {}).get("taps", 0))
        self.side_dim = int((hf.get("token_side") or {}).get("dim", 0))
        self.specs = list(hf["layers"])
        L = len(self.specs)
        self.attn: dict[int, LatentAttention] = {}
        self.rec: dict[int, Hgrn2Mixer] = {}
        self.ff: dict[int, PolyNormMLP | InputScaledMoE] = {}
        self.side: dict[int, TokenSideInput] = {}
        lat = [s["mixer"] for s in self.specs if s["type"] == "latent_attention"]
        # one cache layout for all attention layers: key rows that carry their values (the latent kernel,
        # bf16) when every layer's widths have a kernel shape, else key rows + value columns
        self.latent_cache = dtype == torch.bfloat16 and all(ops.latent_shape(m["kv_rank"], m["rot_dim"]) for m in lat)
        for i, spec in enumerate(self.specs):
            m = spec["mixer"]
            if spec["type"] == "latent_attention":
                src = m.get("kv_from")
                src = i if src is None else int(src)
                if src != i:
                    o = self.specs[src]["mixer"] if 0 <= src < i and self.specs[src]["type"] == "latent_attention" else None
                    if o is None or o.get("kv_from") is not None or (o["kv_rank"], o["rot_dim"]) != (m["kv_rank"], m["rot_dim"]):
                        raise ValueError(f"layer {i}: kv_from {src} must name an earlier latent-attention layer with "
                                         "its own key/value projection and the same kv_rank / rot_dim")
                rot = m["rot"]
                if int(rot.get("dims", m["rot_dim"])) != int(m["rot_dim"]):
                    raise ValueError(f"layer {i}: rot.dims {rot.get('dims')} != rot_dim {m['rot_dim']}")
                self.attn[i] = LatentAttention(i, src, W, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"],
                                               m["q_rank"], rot["base"], rot.get("scaling"), m["scale"], eps, mp,
                                               self.device, dtype, self.latent_cache)
            elif spec["type"] == "hgrn2":
                self.rec[i] = Hgrn2Mixer(W, m["heads"], m["dim"], m["vdim"], eps, self.device, dtype)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {spec['type']!r}")
            f = spec.get("mlp")
            if f:
                kind = f.get("kind", "dense")
                if kind == "dense":
                    self.ff[i] = PolyNormMLP(W, f["ff"], eps, self.device, dtype)
                elif kind == "moe":
                    self.ff[i] = InputScaledMoE(W, f["router"]["experts"], f["router"]["top"], f["expert"]["ff"],
                                                (f.get("shared") or {}).get("ff", 0), self.device, dtype)
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
            if self.side_dim:
                self.side[i] = TokenSideInput(W, self.side_dim, i * self.side_dim, self.device, dtype)
        self.ln1_b: list = [None] * L
        self.ln2_b: list = [None] * L
        self.canon: list = [None] * L          # [W, taps] conv taps of the mixer's input
        self.conv_state: list = [None] * L     # [slots, W, taps - 1] fp32
        self.norm_b = self.side_embed = None
        self.kv_layers = sorted(i for i, a in self.attn.items() if a.own_cache)
        self.kv_heads_per_layer = {i: 1 for i in self.kv_layers}
        self.kv_dims_per_layer = {i: self.attn[i].D for i in self.kv_layers}
        self.kv_value_dim = 0 if self.latent_cache else None      # (0: no value array beside the key rows)
        self.debug_residuals: list | None = None   # set to []: the residual after every layer is appended

    def prefill_item_rows(self, page: int) -> int:
        """Query rows per prefill work item: one plan serves all attention layers, so the 64-row
        item needs every layer to have the shape its kernel is built for."""
        G = LatentAttention.HEAD_GROUP
        rows = {ops.prefill_rows(a.H, 1, a.D, page) if a.H <= G else 32 for a in self.attn.values()}
        return rows.pop() if len(rows) == 1 else 32

    def _blocks(self):
        for d in (self.attn, self.rec, self.ff, self.side):
            yield from d.values()

    def alloc_state(self, slots: int) -> None:
        for b in self._blocks():
            b.alloc_state(slots)
        if self.taps:
            for i in range(len(self.specs)):
                self.conv_state[i] = torch.zeros(slots, self.cfg.hidden_size, max(self.taps - 1, 0),
                                                 dtype=torch.float32, device=self.device)

    # ------------------------------------------------------------------ weights
    def init_random(self, seed: int = 0, std: float = 0.02) -> "MetitarForCausalLM":
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        W, V = self.cfg.hidden_size, self.cfg.vocab_size
        zeros = lambda: torch.zeros(W, dtype=self.dtype, device=self.device)   # noqa: E731
        for i in range(len(self.specs)):
            self.ln1[i], self.ln1_b[i] = self._alloc(W, std=None, gen=gen), zeros()
            if i in self.ff:
                self.ln2[i], self.ln2_b[i] = self._alloc(W, std=None, gen=gen), zeros()
            if self.taps:
                self.canon[i] = self._alloc(W, self.taps, std=0.1, gen=gen)
        for b in self._blocks():
            b.init_random(gen, std)
        self.embed = self._alloc(V, W, std=std, gen=gen)
        if self.side_dim:
            self.side_embed = self._alloc(V, len(self.specs) * self.side_dim, std=1.0, gen=gen)
        self.norm, self.norm_b = self._alloc(W, std=None, gen=gen), zeros()
        self.lm_head = self._alloc(V, W, std=std, gen=gen)
        return self

    def load_hf_weights(self, weights) -> "MetitarForCausalLM":
        put = lambda w: w.to(device=self.device, dtype=self.dtype).contiguous()   # noqa: E731
        top = {"embed": "embed", "side.embed": "side_embed", "final.norm": "norm", "final.norm.b": "norm_b",
               "head": "lm_head"}
        per_layer = {"norm1": self.ln1, "norm1.b": self.ln1_b, "norm2": self.ln2, "norm2.b": self.ln2_b,
                     "canon1": self.canon}
        groups: dict[tuple[int, str], dict[str, torch.Tensor]] = {}
        for name, w in weights:
            if name in top:
                setattr(self, top[name], put(w))
            elif name.startswith("l") and "." in name:
                head, rest = name.split(".", 1)
                if not head[1:].isdigit() or int(head[1:]) >= len(self.specs):
                    continue
                i = int(head[1:])
                if rest in per_layer:
                    per_layer[rest][i] = put(w)
                    continue
                for pre in ("mix.", "mlp.", "side."):
                    if rest.startswith(pre):
                        groups.setdefault((i, pre), {})[rest[len(pre):]] = w
                        break
        for kind, blocks in (("mix.", self.attn), ("mix.", self.rec), ("mlp.", self.ff), ("side.", self.side)):
            for i, b in blocks.items():
                try:
                    b.load(groups.get((i, kind), {}))
                except KeyError as e:
                    raise ValueError(f"checkpoint incomplete: layer {i} {kind}{e.args[0]} is missing") from None
        n = range(len(self.specs))
        missing = [k for k, v in (("embed", self.embed), ("final.norm", self.norm), ("final.norm.b", self.norm_b),
                                  ("head", self.lm_head)) if v is None]
        missing += [f"l{i}.norm1(.b)" for i in n if self.ln1[i] is None or self.ln1_b[i] is None]
        missing += [f"l{i}.norm2(.b)" for i in self.ff if self.ln2[i] is None or self.ln2_b[i] is None]
        missing += [f"l{i}.canon1" for i in n if self.taps and self.canon[i] is None]
        if self.side_dim and self.side_embed is None:
            missing.append("side.embed")
        if missing:
            raise ValueError(f"checkpoint incomplete: {', '.join(missing[:6])} missing")
        for i in n:
            if self.taps and tuple(self.canon[i].shape) != (self.cfg.hidden_size, self.taps):
                raise ValueError(f"l{i}.canon1: shape {tuple(self.canon[i].shape)} != [width, canon.taps]")
        return self

    def weight_bytes(self) -> int:
        own = [self.embed, self.norm, self.norm_b, self.lm_head, self.side_embed]
        own += self.ln1 + self.ln1_b + self.ln2 + self.ln2_b + self.canon
        n = sum(t.numel() * t.element_size() for t in own if t is not None)
        return n + sum(t.numel() * t.element_size() for b in self._blocks() for t in b.tensors())

    def gemm_probe_widths(self):
        return None

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, kv: PagedKVCache,
                input_embeds: torch.Tensor | None = None) -> torch.Tensor:
        """ids [T] int32 -> final normed hidden [T, W] (model dtype)."""
        if input_embeds is not None:
            raise NotImplementedError("Metitar: the per-layer token input needs token ids")
        ctx = MixerCtx(meta, kv, meta.extra["ssm"])
        cu, slot, reset = ctx.seqs
        eps, dt = self.eps, self.dtype
        x = ops.embedding_f32(ids, self.embed, self.embed_scale)          # fp32 stream
        hx = None                                                          # x rounded to the model dtype
        dbg = self.debug_residuals
        for i in range(len(self.specs)):
            if self.taps:
                h = ops.conv_mix(x, self.canon[i], self.conv_state[i], cu, slot, reset, dt)
            else:
                h = hx if hx is not None else x.to(dt)
            y = self.attn[i].forward(h, ctx) if i in self.attn else self.rec[i].forward(h, ctx)
            last = i not in self.ff and i not in self.side
            hx = ops.post_norm_add(x, y, self.ln1[i], self.ln1_b[i], eps, 0, None if last and self.taps else dt)
            if i in self.ff:
                last = i not in self.side
                hx = ops.post_norm_add(x, self.ff[i].forward(hx), self.ln2[i], self.ln2_b[i], eps, 0,
                                       None if last and self.taps else dt)
            if i in self.side:
                s = self.side[i]
                hx = ops.post_norm_add(x, s.forward(hx, ids, self.side_embed), s.norm, None, eps, 1,
                                       None if self.taps else dt)
            if dbg is not None:
                dbg.append(x.clone())
        return ops.row_norm(x, self.norm, self.norm_b, eps, 0)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits: head . hidden * logit_scale."""
        logits = ops.lm_head_f32(hidden, self.lm_head)
        return logits.mul_(self.logit_scale) if self.logit_scale != 1.0 else logits
