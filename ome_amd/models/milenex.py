"""Milenex: a layer-list decoder (``architecture: Milenex``) of attention layers with a token shift
in front of every mixer and an optional looped span of layers.

``layers[i]`` = {``type``, ``mixer`` (that mixer's own sizes), ``mlp`` (or null)}.  Mixer types:

* ``attention`` -- ``mixers.ConvRotaryAttention`` (short causal convolutions on q / k / v, rotary
  pairs, unit-RMS q / k, sliding window, softmax sink);
* ``attention_2`` -- ``mixers.TalkingHeadsAttention`` (logarithmic distance bias, sliding window,
  softmax sink, weights mixed across heads, per-head output gate).

Feed-forwards (``mlp.kind``): ``dense`` = ``mixers.GeluMLP``, ``moe`` = ``mixers.GroupRoutedMoE``.

One layer, with x the fp32 stream and N(x) w = x / rms(x) * (1 + w) (weights stored around zero):

  n = N(x) norm1;  h_t = n_t + (n_{t-1} - n_t) * shift    (n_{-1} = 0: the token shift)
  x += mixer(h);   x += ff(N(x) norm2)

``loop`` = {start, stop, times}: layers start .. stop-1 run ``times`` times in a row with the same
weights; every pass has its own KV pages, conv tails and shift rows, and before every pass but the
first the embedding output is added to x.  x starts as ``embed[token]``; logits = ``head`` . (N(x)
``final.norm``).

Execution is a flat list of layer RUNS (layer, pass); run r owns cache layer r and its own state.
The blocks of later passes are shallow copies of the first pass's blocks: same weight tensors,
their own state.

Numerics: x is fp32 from the embedding to the final norm (``ops.embedding_f32`` ->
``ops.shift_norm``, which adds the previous sublayer's output in fp32, norms, shifts and rounds once
to the model dtype for the next GEMM); the shift rows kept per request slot are the fp32 normed
rows; convolution sums, rotary angles, unit norms, attention scores / weights / mixing, router
logits and scores are fp32 inside the kernels; logits leave the head in fp32.  Prefix caching is
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
from ome_amd.models.mixers import ConvRotaryAttention, GeluMLP, GroupRoutedMoE, MixerCtx, TalkingHeadsAttention
from ome_amd.parallel import state as pstate

MILENEX_ARCHS = {"Milenex"}


class MilenexForCausalLM(LlamaForCausalLM):
    stateful = True
    tune_gemms = False   # odd projection widths: the library heuristic, no TunableOp pass

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16, max_positions: int | None = None):
        st = pstate.get()
        if st.tp_size > 1 or st.pp_size > 1:
            raise NotImplementedError("Milenex: tensor / pipeline parallelism (one GPU holds the model)")
        super().__init__(cfg, device, dtype, 1)   # (the base's rotary table is unused: one row)
        hf = cfg.extra or {}
        W, eps = cfg.hidden_size, cfg.rms_norm_eps
        mp = max_positions or cfg.max_position_embeddings
        self.specs = list(hf["layers"])
        L = len(self.specs)
        self.runs = layer_runs(hf)                       # [(layer, pass)]
        self.loop_start = int((hf.get("loop") or {}).get("start", 0))
        first = {i: r for r, (i, p) in reversed(list(enumerate(self.runs)))}     # layer -> its first run
        self.mix: dict[int, ConvRotaryAttention | TalkingHeadsAttention] = {}     # by RUN
        self.ff: dict[int, GeluMLP | GroupRoutedMoE] = {}                          # by LAYER (stateless)
        for i, spec in enumerate(self.specs):
            if i not in first:
                continue                                  # (a loop that runs zero times)
            m, r = spec["mixer"], first[i]
            if spec["type"] == "attention":
                rot = m.get("rot") or {}
                self.mix[r] = ConvRotaryAttention(r, W, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                                                  m["mask"]["size"], m.get("conv", 0), rot.get("base", 10000.0),
                                                  rot.get("dims", 0), m["scale"], eps, mp, self.device, dtype)
            elif spec["type"] == "attention_2":
                self.mix[r] = TalkingHeadsAttention(r, W, m["heads"], m["kv_heads"], m["dim"], m["vdim"],
                                                    m["mask"]["size"], m["scale"], self.device, dtype)
            else:
                raise ValueError(f"layer {i}: unknown mixer type {spec['type']!r}")
            f = spec.get("mlp")
            if f:
                kind = f.get("kind", "dense")
                if kind == "dense":
                    self.ff[i] = GeluMLP(W, f["ff"], self.device, dtype)
                elif kind == "moe":
                    ro, sh, g = f["router"], f.get("shared") or {}, f["router"].get("groups") or {}
                    self.ff[i] = GroupRoutedMoE(W, ro["experts"], ro["top"], f["expert"]["ff"], f["expert"]["limit"],
                                                int(g.get("count", 1)), int(g.get("keep", 1)), sh.get("ff", 0),
                                                sh.get("limit", 0.0), self.device, dtype)
                else:
                    raise ValueError(f"layer {i}: unknown feed-forward kind {kind!r}")
        self._first = first
        self.shift: list = [None] * L                    # [W] per layer
        self.shift_state: list = [None] * len(self.runs)  # [slots, W] fp32 per run
        self.kv_layers = list(range(len(self.runs)))
        self.debug_residuals: list | None = None   # set to []: the residual after every layer run is appended
        self._set_kv_maps()

    def _set_kv_maps(self) -> None:
        """Every run's cache shape (a later pass has the shape of the first pass's block)."""
        shape = {r: self.mix[self._first[i]] for r, (i, _) in enumerate(self.runs)}
        self.kv_heads_per_layer = {r: b.Hkv for r, b in shape.items()}
        self.kv_dims_per_layer = {r: b.D for r, b in shape.items()}

    def _share_passes(self) -> None:
        """Blocks of later passes: the first pass's weights, their own cache layer and state."""
        for r, (i, p) in enumerate(self.runs):
            if r != self._first[i]:
                b = copy.copy(self.mix[self._first[i]])
                b.layer = r
                self.mix[r] = b

    def prefill_item_rows(self, page: int) -> int:
        """Query rows per prefill work item: one plan serves all attention layers, so the 64-row
        item needs every layer that reads the plan to have the shape its kernel is built for."""
        rows = {ops.prefill_rows(a.Hq, a.Hkv, a.D, page) for a in self.mix.values() if isinstance(a, ConvRotaryAttention)}
        return rows.pop() if len(rows) == 1 else 32

    def _blocks(self):
        first = set(self._first.values())
        yield from (b for r, b in self.mix.items() if r in first)
        yield from self.ff.values()

    def alloc_state(self, slots: int) -> None:
        for b in self.mix.values():
            b.alloc_state(slots)
        for r in range(len(self.runs)):
            self.shift_state[r] = torch.zeros(slots, self.cfg.hidden_size, dtype=torch.float32, device=self.device)

    # ------------------------------------------------------------------ weights
    def init_random(self, seed: int = 0, std: float = 0.02) -> "MilenexForCausalLM":
        gen = torch.Generator(device=self.device)
        gen.manual_seed(seed)
        W, V = self.cfg.hidden_size, self.cfg.vocab_size
        for i in range(len(self.specs)):
            self.ln1[i] = self._alloc(W, std=0.02, gen=gen)
            self.shift[i] = torch.rand(W, generator=gen, device=self.device).to(self.dtype)
            if i in self.ff:
                self.ln2[i] = self._alloc(W, std=0.02, gen=gen)
        for b in self._blocks():
            b.init_random(gen, std)
        self.embed = self._alloc(V, W, std=1.0, gen=gen)
        self.norm = self._alloc(W, std=0.02, gen=gen)
        self.lm_head = self._alloc(V, W, std=std, gen=gen)
        self._share_passes()
        return self

    def load_hf_weights(self, weights) -> "MilenexForCausalLM":
        put = lambda w: w.to(device=self.device, dtype=self.dtype).contiguous()   # noqa: E731
        top = {"embed": "embed", "final.norm": "norm", "head": "lm_head"}
        per_layer = {"norm1": self.ln1, "norm2": self.ln2, "shift": self.shift}
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
        missing = [k for k, v in (("embed", self.embed), ("final.norm", self.norm), ("head", self.lm_head)) if v is None]
        missing += [f"l{i}.norm1 / shift" for i in self._first if self.ln1[i] is None or self.shift[i] is None]
        missing += [f"l{i}.norm2" for i in self.ff if self.ln2[i] is None]
        if missing:
            raise ValueError(f"checkpoint incomplete: {', '.join(missing[:6])} missing")
        self._share_passes()
        return self

    def weight_bytes(self) -> int:
        own = [self.embed, self.norm, self.lm_head] + self.ln1 + self.ln2 + self.shift
        n = sum(t.numel() * t.element_size() for t in own if t is not None)
        return n + sum(t.numel() * t.element_size() for b in self._blocks() for t in b.tensors())

    def gemm_probe_widths(self):
        return None

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, kv: PagedKVCache,
                input_embeds: torch.Tensor | None = None) -> torch.Tensor:
        """ids [T] int32 -> final normed hidden [T, W] (model dtype)."""
        ctx = MixerCtx(meta, kv, meta.extra["ssm"])
        eps, dt = self.eps, self.dtype
        x = ops.embedding_f32(ids, self.embed, 1.0) if input_embeds is None else input_embeds.float()   # fp32 stream
        again = any(p > 0 for _, p in self.runs)
        x0 = (x.clone() if dt == torch.float32 else x.to(dt)) if again else None   # (exact: the table holds dt values)
        pend = None                                  # the sublayer output not yet added to x
        dbg = self.debug_residuals
        for r, (i, p) in enumerate(self.runs):
            extra = x0 if p > 0 and i == self.loop_start else None
            x, h = ops.shift_norm(x, self.ln1[i], eps, pend, 1.0, extra, 1.0, 1.0, self.shift[i],
                                  self.shift_state[r], ctx.seqs, dt)
            pend = self.mix[r].forward(h, ctx)
            if i in self.ff:
                x, h = ops.shift_norm(x, self.ln2[i], eps, pend, w_offset=1.0, out_dtype=dt)
                pend = self.ff[i].forward(h)
            if dbg is not None:
                dbg.append(x + pend.float())
        return ops.shift_norm(x, self.norm, eps, pend, w_offset=1.0, out_dtype=dt)[1]

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        """fp32 logits ``head . hidden``."""
        return ops.lm_head_f32(hidden, self.lm_head)
