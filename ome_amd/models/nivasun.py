"""Nivasun: a layer-list decoder (``architecture: Nivasun``) of parallel blocks -- one norm per
layer, whose output feeds the mixer and the feed-forward side by side -- with a hashed token-pair
embedding, a short causal convolution in front of every mixer and an optional looped span of layers.

``layers[i]`` = {``type``, ``mixer`` (that mixer's own sizes), ``mlp`` (or null)}.  Mixer types:

* ``attention`` -- ``mixers.KeyValuedAttention`` (values = unrotated keys, half-split rotary pairs,
  per-head temperature, sliding window, softmax sink);
* ``attention_2`` -- ``mixers.DifferentialAttention`` (two softmax maps per head over the same
  values, interleaved rotary pairs, sliding window, weightless per-head RMS norm);
* ``latent_attention`` -- ``mixers.LatentAttention`` without a rotated part or sink, with a sliding
  window and a sigmoid output gate.

Feed-forward (``mlp.kind: moe``): ``mixers.GroupRoutedMoE`` as one group of SiLU-GLU experts whose
router has a bias, weighted by the softmax over the chosen logits, plus a gated shared expert.

One layer run, with x the fp32 stream and g_i a single number:

  h  = x / sqrt(mean(x^2) + eps) * g_i                      (``l<i>.norm1``)
  hm = h + causal_conv(h)                                    (``canon.taps`` taps per channel, ``l<i>.canon1``)
  x += mixer(hm) + ff(h)

x starts as ``embed[token] * embedding.scale + bigram[r]``, r = (previous token * mul_prev + token *
mul_cur) mod buckets, the table's extra last row for a sequence's first token.  ``loop`` = {start,
stop, times}: layers start .. stop-1 run ``times`` times in a row with the same weights; every pass
has its own KV pages and conv tails, and right before the first layer of EVERY pass row t of
``loop.step`` is added to x.  logits = cap * tanh(``head`` . norm(x) / cap), cap = ``logit_softcap``.

Execution is a flat list of layer RUNS (layer, pass); run r owns cache layer r and its own state.
The blocks of later passes are shallow copies of the first pass's blocks: same weight tensors,
their own cache layer.

Numerics: x is fp32 from the embedding to the final norm.  ``ops.shift_norm`` (no shift) adds the
two sublayer outputs of the previous run and the pass vector in fp32, norms and rounds once to the
model dtype; the single gain is stored as a row of equal weights so that the stream kernel of the
other layer-list designs serves it.  ``ops.conv_mix`` reads that row and sums in fp32; its tail
state (the last taps - 1 normed rows per request slot and run) is fp32.  Rotary angles, the
temperature, attention scores / softmax / sinks, the head norm of the differential attention, the
latent norms, router logits and weights are fp32 inside the kernels; logits leave the head in fp32.
The previous token of every request slot is part of the state (``prev_token``).  Prefix caching is
off (``stateful``).  The model has no cache, loop over steps or scheduler of its own:
``ModelRunner`` drives it like the other layer-list designs.
"""
from __future__ import annotations

import copy

import torch

from ome_amd import ops
from ome_amd.models.common import AttnMeta, PagedKVCache
from ome_amd.models.config import ModelConfig, layer_runs
from ome_amd.models.llama import LlamaForCausalLM
from ome_amd.models.mixers import (DifferentialAttention, GroupRoutedMoE, KeyValuedAttention, LatentAttention,
                                   MixerCtx)
from ome_amd.parallel import state as pstate

NIVASUN_ARCHS = {"Nivasun"}


class NivasunForCausalLM(LlamaForCausalLM):
    stateful = True
    tune_gemms = False   # odd projection widths: the library heuristic, no TunableOp pass

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16, max_positions: int | None = None):
        st = pstate.get()
        if st.tp_size > 1 or st.pp_size > 1:
            raise NotImplementedError("Nivasun: tensor / pipeline parallelism (one GPU holds the model)")
        super().__init__(cfg, device, dtype, 1)   # (the base's rotary table is unused: one row)
        hf = cfg.extra or {}
        W, eps = cfg.hidden_size, cfg.rms_norm_eps
        mp = max_positions or cfg.max_position_embeddings
        emb = hf.get("embedding") or {}
        self.embed_scale = float(emb.get("scale", 1.0))
        self.pair = dict(emb["bigram"]) if emb.get("bigram") else None      # {buckets, mul_prev, mul_cur}
        self.softcap = float(hf.get("logit_softcap") or 0.0)
        self.taps = int((hf.get("canon") or {}).get("taps", 0))
        self.specs = list(hf["layers"])
        L = len(self.specs)
        self.runs = layer_runs(hf)                       # [(layer, pass)]
        lp = hf.get("loop") or {}
        self.looped = bool(lp) and int(lp.get("stop", 0)) > int(lp.get("start", 0))
        self.loop_start = int(lp.get("start", 0))
        self.loop_times = int(lp.get("times", 1)) if self.looped else 0
        first = {i: r for r, (i, p) in reversed(list(enumerate(self.runs)))}     # layer -> its first run
        lat = [s["mixer"] for s in self.specs if s["type"] == "latent_attention"]
        # key rows that carry their values (the latent kernel, bf16) when every latent layer's width has a
        # kernel shape, else key rows + value columns of the generic kernels
        self.latent_cache = dtype == torch.bfloat16 and bool(lat) and all(ops.latent_shape(m["kv_rank"], 0) for m in lat)
        self.mix: dict[int, KeyValuedAttention | DifferentialAttention | LatentAttention] = {}   # by RUN
        self.ff: dict[int, GroupRoutedMoE] = {}                                                   # by LAYER
        for i, spec in enumerate(self.specs):
            if i not in first:
                continue                                  # (a loop that runs zero times)
            m, r = spec["mixer"], first[i]
            rot = m.get("rot") or {}
            if spec["type"] == "attention":
                if int(m.get("vdim", m["dim"])) != int(m["dim"]):
                    raise ValueError(f"layer {i}: values are the keys, so vdim {m['vdim']} must equal dim {m['dim']}")
                self.mix[r] = KeyValuedAttention(r, W, m["heads"], m["kv_heads"], m["dim"], m["mask"]["size"],
                                                 rot.get("base", 10000.0), rot.get("dims", 0), m["scale"], mp,
                                                 self.device, dtype)
            elif spec["type"] == "attention_2":
                self.mix[r] = DifferentialAttention(r, W, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                                                    m["mask"]["size"], rot.get("base", 10000.0), rot.get("dims", 0),
                                                    m["scale"], m["diff"], eps, mp, self.device, dtype)
            elif spec["type"] == "latent_attention":
                self.mix[r] = LatentAttention(r, r, W, m["heads"], m["dim"], 0, m["vdim"], m["kv_rank"], m["q_rank"],
                                              1.0, None, m["scale"], eps, mp, self.device, dtype, self.latent_cache,
                                              window=m["mask"]["size"], sink=False, gated=True)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {spec['type']!r}")
            f = spec.get("mlp")
            if f:
                if f.get("kind", "moe") != "moe":
                    raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
                ro, sh = f["router"], f.get("shared") or {}
                self.ff[i] = GroupRoutedMoE(W, ro["experts"], ro["top"], f["expert"]["ff"], 0.0, 1, 1, sh.get("ff", 0),
                                            0.0, self.device, dtype, act=0, renorm=True, router_bias=True,
                                            correction=False)
        self._first = first
        self.canon: list = [None] * L                    # [W, taps] conv taps of the mixer's input
        self.conv_state: list = [None] * len(self.runs)   # [slots, W, taps - 1] fp32 per run
        self.pair_table = self.loop_step = None
        self.prev_token = None                           # [slots] int32: every request's last token
        self.kv_layers = list(range(len(self.runs)))
        self.debug_residuals: list | None = None   # set to []: the residual after every layer run is appended
        self._set_kv_maps()

    def _set_kv_maps(self) -> None:
        """Every run's cache shape (a later pass has the shape of the first pass's block)."""
        shape = {r: self.mix[self._first[i]] for r, (i, _) in enumerate(self.runs)}
        self.kv_heads_per_layer = {r: 1 if isinstance(b, LatentAttention) else b.Hkv for r, b in shape.items()}
        self.kv_dims_per_layer = {r: b.D for r, b in shape.items()}
        # (a latent layer's key rows carry their values: no value array)
        self.kv_value_dim = {r: 0 if isinstance(b, LatentAttention) and b.latent_cache else b.D for r, b in shape.items()}
        # fewest kv heads among the layers that run the split-K decode kernel (latent layers on the latent
        # kernel bring their own workspace): the runner partitions its decode workspace by it
        paged = [self.kv_heads_per_layer[r] for r, b in shape.items() if not (isinstance(b, LatentAttention) and b.latent_cache)]
        self.decode_ws_kv_heads = min(paged) if paged else None

    def _share_passes(self) -> None:
        """Blocks of later passes: the first pass's weights, their own cache layer."""
        for r, (i, p) in enumerate(self.runs):
            if r != self._first[i]:
                b = copy.copy(self.mix[self._first[i]])
                b.layer = r
                if isinstance(b, LatentAttention):
                    b.kv_layer = r
                self.mix[r] = b

    def prefill_item_rows(self, page: int) -> int:
        """Query rows per prefill work item: one plan serves all attention layers, so the 64-row
        item needs every layer that reads the plan to have the shape its kernel is built for."""
        rows = set()
        for a in self.mix.values():
            if isinstance(a, LatentAttention):
                if not a.latent_cache:
                    rows.add(ops.prefill_rows(a.H, 1, a.D, page) if a.H <= LatentAttention.HEAD_GROUP else 32)
            else:
                rows.add(ops.prefill_rows(a.Hq, a.Hkv, a.D, page))
        return rows.pop() if len(rows) == 1 else 32

    def _blocks(self):
        first = set(self._first.values())
        yield from (b for r, b in self.mix.items() if r in first)
        yield from self.ff.values()

    def alloc_state(self, slots: int) -> None:
        for b in self.mix.values():
            b.alloc_state(slots)
        if self.taps:
            for r in range(len(self.runs)):
                self.conv_state[r] = torch.zeros(slots, self.cfg.hidden_size, self.taps - 1, dtype=torch.float32,
                                                 device=self.device)
        self.prev_token = torch.zeros(slots, dtype=torch.int32, device=self.device)

    # ------------------------------------------------------------------ weights
    def _gain(self, g: torch.Tensor) -> torch.Tensor:
        """A norm's single gain as a weight row (all entries equal)."""
        if g.numel() != 1:
            raise ValueError(f"norm gain: one number expected, got shape {tuple(g.shape)}")
        return g.reshape(1).to(device=self.device, dtype=self.dtype).expand(self.cfg.hidden_size).contiguous()

    def init_random(self, seed: int = 0, std: float = 0.02) -> "NivasunForCausalLM":
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        W, V = self.cfg.hidden_size, self.cfg.vocab_size
        one = torch.ones((), dtype=self.dtype)
        for i in range(len(self.specs)):
            self.ln1[i] = self._gain(one)
            if self.taps:
                self.canon[i] = self._alloc(W, self.taps, std=0.1, gen=gen)
        for b in self._blocks():
            b.init_random(gen, std)
        self.embed = self._alloc(V, W, std=1.0 / max(self.embed_scale, 1e-6), gen=gen)
        if self.pair:
            self.pair_table = self._alloc(int(self.pair["buckets"]) + 1, W, std=0.5, gen=gen)
        if self.looped:
            self.loop_step = self._alloc(self.loop_times, W, std=0.1, gen=gen)
        self.norm = self._gain(one)
        self.lm_head = self._alloc(V, W, std=std, gen=gen)
        self._share_passes()
        return self

    def load_hf_weights(self, weights) -> "NivasunForCausalLM":
        put = lambda w: w.to(device=self.device, dtype=self.dtype).contiguous()   # noqa: E731
        top = {"embed": "embed", "bigram": "pair_table", "loop.step": "loop_step", "head": "lm_head"}
        groups: dict[tuple[int, str], dict[str, torch.Tensor]] = {}
        for name, w in weights:
            if name in top:
                setattr(self, top[name], put(w))
            elif name == "final.norm":
                self.norm = self._gain(w)
            elif name.startswith("l") and "." in name:
                head, rest = name.split(".", 1)
                if not head[1:].isdigit() or int(head[1:]) >= len(self.specs):
                    continue
                i = int(head[1:])
                if rest == "norm1":
                    self.ln1[i] = self._gain(w)
                elif rest == "canon1":
                    self.canon[i] = put(w)
                else:
                    for pre in ("mix.", "mlp."):
                        if rest.startswith(pre):
                            groups.setdefault((i, pre), {})[rest[len(pre):]] = w
                            break
        for i, r in self._first.items():
            for kind, b in (("mix.", self.mix[r]), ("mlp.", self.ff.get(i))):
                if b is None:
                    continue
                try:
                    b.load(groups.get((i, kind), {}))
                except KeyError as e:
                    raise ValueError(f"checkpoint incomplete: l{i}.{kind}{e.args[0]} is missing") from None
        W = self.cfg.hidden_size
        missing = [k for k, v in (("embed", self.embed), ("final.norm", self.norm), ("head", self.lm_head)) if v is None]
        missing += [f"l{i}.norm1" for i in self._first if self.ln1[i] is None]
        missing += [f"l{i}.canon1" for i in self._first if self.taps and self.canon[i] is None]
        if self.pair and self.pair_table is None:
            missing.append("bigram")
        if self.looped and self.loop_step is None:
            missing.append("loop.step")
        if missing:
            raise ValueError(f"checkpoint incomplete: {', '.join(missing[:6])} missing")
        for i in self._first:
            if self.taps and tuple(self.canon[i].shape) != (W, self.taps):
                raise ValueError(f"l{i}.canon1: shape {tuple(self.canon[i].shape)} != [width, canon.taps]")
        if self.pair and tuple(self.pair_table.shape) != (int(self.pair["buckets"]) + 1, W):
            raise ValueError(f"bigram: shape {tuple(self.pair_table.shape)} != [buckets + 1, width]")
        if self.looped and tuple(self.loop_step.shape) != (self.loop_times, W):
            raise ValueError(f"loop.step: shape {tuple(self.loop_step.shape)} != [times, width]")
        self._share_passes()
        return self

    def weight_bytes(self) -> int:
        own = [self.embed, self.norm, self.lm_head, self.pair_table, self.loop_step] + self.ln1 + self.canon
        n = sum(t.numel() * t.element_size() for t in own if t is not None)
        return n + sum(t.numel() * t.element_size() for b in self._blocks() for t in b.tensors())

    def gemm_probe_widths(self):
        return None

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, kv: PagedKVCache,
                input_embeds: torch.Tensor | None = None) -> torch.Tensor:
        """ids [T] int32 -> final normed hidden [T, W] (model dtype)."""
        if input_embeds is not None:
            raise NotImplementedError("Nivasun: the token-pair embedding needs token ids")
        ctx = MixerCtx(meta, kv, meta.extra["ssm"])
        cu, slot, reset = ctx.seqs
        eps, dt = self.eps, self.dtype
        if self.pair:
            x = ops.pair_embedding_f32(ids, self.embed, self.embed_scale, self.pair_table, int(self.pair["buckets"]),
                                       int(self.pair["mul_prev"]), int(self.pair["mul_cur"]), self.prev_token, ctx.seqs)
        else:
            x = ops.embedding_f32(ids, self.embed, self.embed_scale)          # fp32 stream
        y1 = y2 = None                               # the sublayer outputs not yet added to x
        dbg = self.debug_residuals
        for r, (i, p) in enumerate(self.runs):
            step = self.loop_step[p] if self.looped and i == self.loop_start else None
            x, h = ops.shift_norm(x, self.ln1[i], eps, y1, 1.0, y2, 1.0, out_dtype=dt, bias=step)
            hm = ops.conv_mix(h, self.canon[i], self.conv_state[r], cu, slot, reset, dt) if self.taps else h
            y1 = self.mix[r].forward(hm, ctx)
            y2 = self.ff[i].forward(h) if i in self.ff else None
            if dbg is not None:
                dbg.append(x + y1.float() + (y2.float() if y2 is not None else 0.0))
        return ops.shift_norm(x, self.norm, eps, y1, 1.0, y2, 1.0, out_dtype=dt)[1]

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits ``cap * tanh(head . hidden / cap)`` (no cap: the plain product)."""
        logits = ops.lm_head_f32(hidden, self.lm_head)
        if self.softcap > 0:
            logits = torch.tanh(logits.div_(self.softcap)).mul_(self.softcap)
        return logits
