"""Zavilorn: a decoder whose config lists its layers one by one (``architecture: Zavilorn``).

``layers[i]`` = {``type``, ``mixer`` (that mixer's own sizes), ``mlp`` (or null)}; sizes may differ
from layer to layer.  Layer types:

* ``parallel`` -- two mixers read the same normed input side by side: a gated sliding-window
  attention that keeps the first tokens visible (``mixers.GatedWindowAttention``, ``mixer.left``)
  and a gated delta rule (``mixers.GatedDeltaMixer``, ``mixer.right``); the block's output is
  ``left_scale * left + right_scale * right``;
* ``mamba2`` -- ``mixers.Mamba2Mixer``.

Every block is pre-norm: x += mixer(rmsnorm(x) w1), then (if the layer has one) x += ff(rmsnorm(x)
w2) with the clamped GLU ``mixers.ClampedGLU``.  x starts as ``embed[token] * embedding.scale``;
logits = embed . (rmsnorm(x) w_final) with the unscaled table.

Numerics: the residual stream x is fp32 for the whole stack (``ops.embedding_f32`` ->
``ops.residual_rmsnorm``, which adds the previous sublayer's output(s) in fp32 and emits the
normed GEMM input in the model dtype); projections run in the model dtype with fp32 accumulation;
attention logits / softmax, norms, rotary angles, decays, gates of the recurrences and both
recurrent states are fp32 inside the kernels.  Logits leave the LM head in fp32.

Cache and state: only ``parallel`` layers own KV pages (``kv_layers``), each with its own kv-head
count and head width (``kv_heads_per_layer`` / ``kv_dims_per_layer``; widths padded to the 64 /
128 / 256 kernel tile); the recurrent layers keep conv tails and fp32 states per request slot
(``alloc_state``).  Prefix caching is off (``stateful``).  Checkpoint names: ``embed``,
``final.norm``, ``l<i>.norm1|norm2``, ``l<i>.mix.*`` (``.left.`` / ``.right.`` inside a parallel
block), ``l<i>.mlp.*``.
"""
from __future__ import annotations

import torch

from ome_amd import ops
from ome_amd.models.common import AttnMeta, PagedKVCache
from ome_amd.models.config import ModelConfig
from ome_amd.models.llama import LlamaForCausalLM
from ome_amd.models.mixers import ClampedGLU, GatedDeltaMixer, GatedWindowAttention, Mamba2Mixer, MixerCtx
from ome_amd.parallel import state as pstate

ZAVILORN_ARCHS = {"Zavilorn"}


class ZavilornForCausalLM(LlamaForCausalLM):
    stateful = True
    tune_gemms = False   # odd projection widths: the library heuristic, no TunableOp pass

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16, max_positions: int | None = None):
        st = pstate.get()
        if st.tp_size > 1 or st.pp_size > 1:
            raise NotImplementedError("Zavilorn: tensor / pipeline parallelism (one GPU holds the model)")
        super().__init__(cfg, device, dtype, 1)   # (the base's rotary table is unused: one row)
        hf = cfg.extra or {}
        W, eps = cfg.hidden_size, cfg.rms_norm_eps
        mp = max_positions or cfg.max_position_embeddings
        self.embed_scale = float((hf.get("embedding") or {}).get("scale", 1.0))
        self.specs = list(hf["layers"])
        self.left: dict[int, GatedWindowAttention] = {}
        self.right: dict[int, GatedDeltaMixer] = {}
        self.mamba: dict[int, Mamba2Mixer] = {}
        self.ff: dict[int, ClampedGLU] = {}
        self.mix_scale: dict[int, tuple[float, float]] = {}
        for i, L in enumerate(self.specs):
            m = L["mixer"]
            if L["type"] == "parallel":
                a, r = m["left"], m["right"]
                self.left[i] = GatedWindowAttention(
                    i, W, a["heads"], a["kv_heads"], a["dim"], a["vdim"], a["mask"]["size"], a["mask"]["keep_first"],
                    a["rot"]["base"], a["rot"]["dims"], a["scale"], eps, mp, self.device, dtype)
                self.right[i] = GatedDeltaMixer(W, r["heads"], r["kv_heads"], r["dim"], r["vdim"], r["conv"], eps,
                                                self.device, dtype)
                self.mix_scale[i] = (float(m["left_scale"]), float(m["right_scale"]))
            elif L["type"] == "mamba2":
                self.mamba[i] = Mamba2Mixer(W, m["heads"], m["vdim"], m["state"], m["groups"], m["conv"],
                                            m["norm_groups"], eps, self.device, dtype)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {L['type']!r}")
            f = L.get("mlp")
            if f:
                if f.get("kind", "dense") != "dense":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
                self.ff[i] = ClampedGLU(W, f["ff"], f["limit"], self.device, dtype)
        self.kv_layers = sorted(self.left)
        self.kv_heads_per_layer = {i: a.Hkv for i, a in self.left.items()}
        self.kv_dims_per_layer = {i: a.D for i, a in self.left.items()}
        self.debug_residuals: list | None = None   # set to []: the residual after every layer is appended

    def prefill_item_rows(self, page: int) -> int:
        """Query rows per prefill work item: one plan serves all attention layers, so the 64-row
        item needs every layer to have the shape its kernel is built for."""
        rows = {32 if a.keep_first > 0 else ops.prefill_rows(a.Hq, a.Hkv, a.D, page) for a in self.left.values()}
        return rows.pop() if len(rows) == 1 else 32

    def _blocks(self):
        for d in (self.left, self.right, self.mamba, self.ff):
            yield from d.values()

    def alloc_state(self, slots: int) -> None:
        for b in self._blocks():
            b.alloc_state(slots)

    # ------------------------------------------------------------------ weights
    def init_random(self, seed: int = 0, std: float = 0.02) -> "ZavilornForCausalLM":
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        W = self.cfg.hidden_size
        for i in range(len(self.specs)):
            self.ln1[i] = self._alloc(W, std=None, gen=gen)
            if i in self.ff:
                self.ln2[i] = self._alloc(W, std=None, gen=gen)
        for b in self._blocks():
            b.init_random(gen, std)
        self.embed = self._alloc(self.cfg.vocab_size, W, std=std, gen=gen)
        self.norm = self._alloc(W, std=None, gen=gen)
        self.lm_head = self.embed
        return self

    def load_hf_weights(self, weights) -> "ZavilornForCausalLM":
        groups: dict[tuple[int, str], dict[str, torch.Tensor]] = {}
        for name, w in weights:
            if name == "embed":
                self.embed = w.to(device=self.device, dtype=self.dtype).contiguous()
            elif name == "final.norm":
                self.norm = w.to(device=self.device, dtype=self.dtype).contiguous()
            elif name.startswith("l") and "." in name:
                head, rest = name.split(".", 1)
                if not head[1:].isdigit():
                    continue
                i = int(head[1:])
                if rest in ("norm1", "norm2"):
                    (self.ln1 if rest == "norm1" else self.ln2)[i] = w.to(device=self.device, dtype=self.dtype)
                    continue
                for pre in ("mix.left.", "mix.right.", "mix.", "mlp."):
                    if rest.startswith(pre):
                        groups.setdefault((i, pre), {})[rest[len(pre):]] = w
                        break
        for kind, blocks in (("mix.left.", self.left), ("mix.right.", self.right), ("mix.", self.mamba),
                             ("mlp.", self.ff)):
            for i, b in blocks.items():
                try:
                    b.load(groups.get((i, kind), {}))
                except KeyError as e:
                    raise ValueError(f"checkpoint incomplete: layer {i} {kind}{e.args[0]} is missing") from None
        if self.embed is None or self.norm is None or any(self.ln1[i] is None for i in range(len(self.specs))):
            raise ValueError("checkpoint incomplete: embed / final.norm / norm1 missing")
        self.lm_head = self.embed
        return self

    def weight_bytes(self) -> int:
        n = sum(t.numel() * t.element_size() for t in [self.embed, self.norm] + self.ln1 + self.ln2 if t is not None)
        return n + sum(t.numel() * t.element_size() for b in self._blocks() for t in b.tensors())

    def gemm_probe_widths(self):
        return None

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, kv: PagedKVCache,
                input_embeds: torch.Tensor | None = None) -> torch.Tensor:
        """ids [T] int32 -> final normed hidden [T, W] (model dtype)."""
        ctx = MixerCtx(meta, kv, meta.extra["ssm"])
        eps = self.eps
        x = ops.embedding_f32(ids, self.embed, self.embed_scale) if input_embeds is None else input_embeds.float()
        pend: tuple = (None, 1.0, None, 1.0)    # sublayer outputs not yet added to x: (x1, s1, x2, s2)
        dbg = self.debug_residuals
        for i in range(len(self.specs)):
            h = ops.residual_rmsnorm(x, self.ln1[i], eps, *pend, out_dtype=self.dtype)
            if i in self.left:
                ls, rs = self.mix_scale[i]
                pend = (self.left[i].forward(h, ctx), ls, self.right[i].forward(h, ctx), rs)
            else:
                pend = (self.mamba[i].forward(h, ctx), 1.0, None, 1.0)
            if i in self.ff:
                h = ops.residual_rmsnorm(x, self.ln2[i], eps, *pend, out_dtype=self.dtype)
                pend = (self.ff[i].forward(h), 1.0, None, 1.0)
            if dbg is not None:
                r = x + pend[1] * pend[0].float()
                dbg.append(r if pend[2] is None else r + pend[3] * pend[2].float())
        return ops.residual_rmsnorm(x, self.norm, eps, *pend, out_dtype=self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits against the (unscaled) embedding table."""
        return ops.lm_head_f32(hidden, self.lm_head)
