"""Token mixers and feed-forwards as parameterised building blocks (every size and constant is a
constructor argument), for decoders that assemble their layers from a per-layer list.

* :class:`GatedWindowAttention` -- grouped-query attention over the paged KV cache with a sliding
  window that keeps the sequence's first tokens visible, projection-wide q / k RMSNorm, partial
  rotary embedding (interleaved or half-split pairs) and a sigmoid output gate;
* :class:`GatedDeltaMixer` -- the gated delta rule (short causal convolutions, unit-norm q / k,
  per-head decay and write strength, fp32 state per request slot);
* :class:`Mamba2Mixer` -- Mamba-2 / SSD selective scan with grouped B / C and a gated group norm;
* :class:`ClampedGLU` -- gated feed-forward ``min(g, L) * sigmoid(1.702 min(g, L)) * (clamp(u, -L, L) + 1)``;
* :class:`LatentAttention` -- multi-head latent attention (low-rank queries, one cached latent +
  one shared rotary key per token, YaRN-scaled rotary table, a learned per-head softmax sink), run
  absorbed as multi-query attention over the paged cache; a layer may read another layer's cache;
* :class:`Hgrn2Mixer` -- HGRN2 gated linear recurrence (lower-bounded forget gate that also sets
  the write strength, fp32 state per request slot, per-head RMS norm);
* :class:`PolyNormMLP` -- two-matrix feed-forward with the PolyNorm activation;
* :class:`InputScaledMoE` -- sigmoid-routed mixture of SwiGLU experts whose router score scales the
  expert's input, plus an optional always-on shared expert;
* :class:`TokenSideInput` -- a gated per-layer slice of a second token embedding, projected back to
  the stream;
* :class:`KeyValuedAttention` -- grouped-query attention whose values are the unrotated keys, with
  a per-head temperature, a sliding window and a softmax sink;
* :class:`DifferentialAttention` -- two softmax maps per head over the same values, the second
  taken off the first, then a weightless per-head RMS norm.

Each block owns its weights (fused input projection, checkpoint tensors concatenated at load), its
recurrent state (``alloc_state``) and one ``forward(h, ctx)`` over a varlen batch of rows: prompt
chunks and single decode rows alike, described by :class:`MixerCtx`.  The projections run on the
framework's GEMM dispatch (``quant.linear``); everything between them is one of the HIP ops of
``ome_amd.ops`` (CPU tensors: their fp32 references).
"""
from __future__ import annotations

import math
from dataclasses import dataclass, field

import torch

from ome_amd import ops
from ome_amd.models.common import AttnMeta, PagedKVCache, mixed_attention
from ome_amd.models.config import attn_tile_dim, latent_row_width, plain_rope_table, yarn_rope_table
from ome_amd.models.quant import linear


@dataclass
class MixerCtx:
    """One step's batch as the mixers see it: attention metadata + paged cache for the layers that
    own KV pages, ``seqs`` = (cu, slot, reset) row ranges / state slots / fresh-start flags for the
    recurrent ones."""
    meta: AttnMeta
    kv: PagedKVCache
    seqs: tuple
    cache: dict = field(default_factory=dict)   # tensors derived once per step and shared by the layers


MAX_HEAD_GROUP = 16   # query heads per kv head one launch of the paged attention kernels takes


def paged_attention(q: torch.Tensor, k_cache, v_cache, meta: AttnMeta, scale: float, window: int = -1,
                    keep_first: int = 0, sinks: torch.Tensor | None = None) -> torch.Tensor:
    """Decode / prefill / mixed dispatch over the paged cache (q [T, Hq, D] -> [T, Hq, D]).
    ``sinks``: fp32 [Hq] logits that join each head's softmax denominator (no key, no value).
    More than ``MAX_HEAD_GROUP`` query heads per kv head run as several launches over slices of
    every kv head's group."""
    T, Hq, D = q.shape
    Hkv = k_cache.shape[1]
    R = Hq // Hkv
    if R > MAX_HEAD_GROUP and q.is_contiguous():
        q4 = q.view(T, Hkv, R, D)
        out = torch.empty_like(q4)
        for c in range(0, R, MAX_HEAD_GROUP):
            e = min(R, c + MAX_HEAD_GROUP)
            sk = None if sinks is None else sinks.view(Hkv, R)[:, c:e].reshape(-1).contiguous()
            part = paged_attention(q4[:, :, c:e].reshape(T, Hkv * (e - c), D).contiguous(), k_cache, v_cache, meta, scale, window,
                                   keep_first, sk)
            out[:, :, c:e] = part.view(T, Hkv, e - c, D)
        return out.view(T, Hq, D)
    kw = dict(window=window, keep_first=keep_first, sinks=sinks)
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


class LatentAttention(_Block):
    """Multi-head latent attention.  c_q = RMSNorm(W_dq h) w_dqn, q = W_uq c_q, laid out per head
    as [``dim`` unrotated | ``rot_dim`` rotated]; W_dkv h = [``kv_rank`` latent | ``rot_dim`` shared
    rotary key]; c = RMSNorm(latent) w_dkvn; per head k = [W_uk c | rope(k_pe)], v = W_uv c; score =
    q . k * ``scale``; causal softmax whose denominator also holds exp(``sink``_h); W_o.  Rotary
    pairs are (i, i + rot_dim/2) with the YaRN-scaled table of ``config.yarn_rope_table``.

    Runs absorbed: q_lat = W_uk^T q_nope, so all heads share one key [c | rope(k_pe)] and one value
    c per token -- multi-query attention over one cached row per token, whatever the head count.
    Two cache layouts (``latent_cache``, chosen by the model for all its layers):

    * key rows that carry their own values, ``[c | 0 .. | rope(k_pe) | 0 ..]`` in one of the widths of
      ``ops.LATENT_SHAPES`` (bf16): ``ops.latent_prep`` -> ``ops.latent_attn`` (the 16-head MFMA latent
      kernel: one launch for prompt chunks, decode rows and mixed batches) -> W_uv per head;
    * key rows + value columns of the generic paged attention kernels, head width
      ``config.latent_row_width`` (fp32 models, and widths the latent kernel is not built for):
      ``ops.latent_prep`` -> ``paged_attention`` (more than 16 heads in groups of 16) -> W_uv.

    ``kv_layer`` != ``layer``: this layer has no W_dkv and attends over ``kv_layer``'s cache rows with
    its own W_uk / W_uv.  ``rot_dim`` = 0: no rotated part at all (no positions).  ``window`` > 0:
    query i sees keys j with 0 <= i - j < window.  ``sink`` False: an ordinary softmax.  ``gated``:
    the concatenated heads are multiplied by sigmoid(W_g h) before W_o (W_g rides in the fused
    input projection).  Checkpoint tensors ``dq dq.norm uq [dkv dkv.norm] uk uv [sink] [g] o``."""

    HEAD_GROUP = 16   # query heads per kv head one launch of the generic attention kernels takes

    def __init__(self, layer: int, kv_layer: int, width: int, heads: int, dim: int, rot_dim: int, vdim: int,
                 kv_rank: int, q_rank: int, rot_base: float, rot_scaling: dict | None, scale: float, eps: float,
                 max_positions: int, device, dtype, latent_cache: bool | None = None, window: int = -1,
                 sink: bool = True, gated: bool = False):
        super().__init__(device, dtype)
        if rot_dim % 2 or rot_dim < 0:
            raise ValueError(f"latent attention: rotary width {rot_dim} must be even")
        self.window, self.has_sink, self.gated = int(window) if window and window > 0 else -1, bool(sink), bool(gated)
        self.layer, self.kv_layer, self.width, self.H = layer, kv_layer, width, heads
        self.dim, self.rot, self.vdim, self.R, self.qr = dim, rot_dim, vdim, kv_rank, q_rank
        self.scale, self.eps = float(scale), float(eps)
        self.own_cache = kv_layer == layer
        shape = ops.latent_shape(kv_rank, rot_dim) if dtype == torch.bfloat16 else None
        self.latent_cache = shape is not None if latent_cache is None else bool(latent_cache)
        if self.latent_cache:
            if shape is None:
                raise ValueError(f"latent attention: no latent kernel for a {kv_rank} + {rot_dim}-wide row in {dtype}")
            self.D, self.DV = shape              # row width, value width (= where the rotary key starts)
        else:
            self.D = latent_row_width(kv_rank, rot_dim)
            self.DV = kv_rank
            if dtype != torch.float32 and self.D > 256:
                raise ValueError(f"latent attention: a {kv_rank} + {rot_dim}-wide row fits neither the latent kernel "
                                 "(latent <= 512, rotary <= 64) nor the 256-wide attention tile")
        self.cos_sin = yarn_rope_table(rot_base, rot_dim, max_positions, rot_scaling, self.device) if rot_dim else \
            torch.zeros(max_positions, 0, device=self.device)
        self.w_in = self.qn = self.w_uq = self.kvn = self.w_uk = self.w_uv = self.sink = self.w_o = None

    def load(self, t: dict) -> None:
        H, R = self.H, self.R
        parts = [t["dq"]] + ([t["dkv"]] if self.own_cache else []) + ([t["g"]] if self.gated else [])
        self.w_in = self._put(torch.cat(parts, 0))
        self.qn, self.w_uq = self._put(t["dq.norm"]), self._put(t["uq"])
        if self.own_cache:
            self.kvn = self._put(t["dkv.norm"])
        self.w_uk = self._put(t["uk"].view(H, self.dim, R))                       # q_lat = q_nope @ W_uk[h]
        self.w_uv = self._put(t["uv"].view(H, self.vdim, R).transpose(1, 2))      # o = o_lat @ W_uv[h]^T
        self.sink = self._put(t["sink"], torch.float32) if self.has_sink else None
        self.w_o = self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        H, R = self.H, self.R
        self.w_in = self._rand(gen, self.qr + (R + self.rot if self.own_cache else 0) +
                               (H * self.vdim if self.gated else 0), self.width, std=std)
        self.qn = torch.ones(self.qr, dtype=self.dtype, device=self.device)
        self.w_uq = self._rand(gen, H * (self.dim + self.rot), self.qr, std=std)
        if self.own_cache:
            self.kvn = torch.ones(R, dtype=self.dtype, device=self.device)
        self.w_uk, self.w_uv = self._rand(gen, H, self.dim, R, std=std), self._rand(gen, H, R, self.vdim, std=std)
        self.sink = torch.zeros(H, dtype=torch.float32, device=self.device) if self.has_sink else None
        self.w_o = self._rand(gen, self.width, H * self.vdim, std=std)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        T, H, R, D = h.shape[0], self.H, self.R, self.D
        a = linear(h, self.w_in)                                          # [T, q_rank (| latent | k_pe)]
        q = linear(ops.row_norm(a[:, :self.qr], self.qn, None, self.eps, 1), self.w_uq).view(T, H, self.dim + self.rot)
        q_full = torch.empty(T, H, D, dtype=h.dtype, device=h.device)     # [W_uk^T q_nope | 0 | rope(q_pe) | 0]
        k_cache, v_cache = ctx.kv.layer(self.kv_layer)
        own = self.own_cache
        ops.latent_prep(a, self.qr, R, self.rot, self.kvn, self.eps, ctx.meta.positions, self.cos_sin, ctx.meta.slots,
                        k_cache if own else None, v_cache if own and not self.latent_cache else None, q, self.dim,
                        q_full, rope_off=self.DV)
        torch.bmm(q[..., :self.dim].transpose(0, 1), self.w_uk, out=q_full[:, :, :R].transpose(0, 1))
        if self.latent_cache:
            o_lat = torch.empty(T, H, self.DV, dtype=h.dtype, device=h.device)
            rows3 = k_cache.view(k_cache.shape[0], k_cache.shape[2], D)
            ws = _latent_workspace(h)
            for s, e, bt, rows, lens in latent_rows(ctx.meta, T):
                ops.latent_attn(q_full[s:e], rows3, bt, rows, lens, self.scale, self.DV, ws, out=o_lat[s:e],
                                sinks=self.sink, window=self.window)
        else:
            G = self.HEAD_GROUP
            if H <= G:
                o_lat = paged_attention(q_full, k_cache, v_cache, ctx.meta, self.scale, self.window, sinks=self.sink)
            else:   # the kernels share one kv head among at most G query heads: run the heads in groups
                o_lat = torch.cat([paged_attention(q_full[:, g:g + G], k_cache, v_cache, ctx.meta, self.scale,
                                                   self.window, sinks=None if self.sink is None else self.sink[g:g + G])
                                   for g in range(0, H, G)], 1)
        o = torch.empty(T, H * self.vdim, dtype=h.dtype, device=h.device)
        torch.bmm(o_lat[:, :, :R].transpose(0, 1), self.w_uv, out=o.view(T, H, self.vdim).transpose(0, 1))
        if self.gated:
            o = ops.head_gate(o.view(T, H, self.vdim), a[:, a.shape[1] - H * self.vdim:], self.vdim, 0)
        return linear(o, self.w_o)


_ARANGE: dict = {}
_ARANGE_KEEP: list = []
_LATENT_WS: dict = {}


def latent_rows(meta: AttnMeta, T: int) -> list:
    """The step's rows as the latent attention kernel takes them: segments (first row, end row,
    block table, block-table row per token, visible keys per token) -- one for the prompt chunks,
    one for the single decode rows of a mixed step."""
    dev = meta.positions.device
    ar = _ARANGE.get(dev)
    if ar is None or ar.numel() < T:
        ar = _ARANGE[dev] = torch.arange(max(T, 4096), dtype=torch.int32, device=dev)
        _ARANGE_KEEP.append(ar)    # (captured decode graphs keep reading the one they were recorded with)
    if meta.is_decode:
        return [(0, T, meta.block_tables, ar[:T], meta.seq_lens)]
    kv_lens = (meta.positions + 1).to(torch.int32)
    n = meta.num_prefill if meta.mode == "mixed" else T
    seg = []
    if n:
        cu = meta.cu_q
        rows = torch.searchsorted(cu[1:].contiguous(), ar[:n].to(cu.dtype), right=True).to(torch.int32)
        seg.append((0, n, meta.block_tables, rows, kv_lens[:n]))
    if n < T:
        seg.append((n, T, meta.dec_block_tables, ar[:T - n], meta.seq_lens))
    return seg


def _latent_workspace(x: torch.Tensor):
    """Split-K partials of the latent kernel, one per stream (layers of a stream run in turn)."""
    if not x.is_cuda:
        return None
    key = (x.device, torch.cuda.current_stream(x.device).cuda_stream)
    ws = _LATENT_WS.get(key)
    if ws is None:
        ws = _LATENT_WS[key] = ops.MLAWorkspace(x.device)
    return ws


class Hgrn2Mixer(_Block):
    """HGRN2.  q = silu(W_q h) (``heads`` x ``dim``), v = W_v h (``heads`` x ``vdim``), forget gate
    f = l + (1 - l) sigmoid(W_f h + b_f) with the learned lower bound l; per head S <- diag(f) S +
    (1 - f) v^T, o = S^T q (no key, no other scale); RMSNorm of each head's o with a shared weight
    [vdim]; W_o.  Checkpoint tensors ``q f f.b lower v norm o``; state S [slots, heads, dim, vdim]
    fp32.  Activations, gate, recurrence and norm are one kernel (``ops.hgrn2_scan``)."""

    def __init__(self, width: int, heads: int, dim: int, vdim: int, eps: float, device, dtype):
        super().__init__(device, dtype)
        self.width, self.H, self.dim, self.vdim, self.eps = width, heads, dim, vdim, float(eps)
        self.w_in = self.f_bias = self.lower = self.gnorm = self.w_o = None
        self.rec_state = None

    def load(self, t: dict) -> None:
        self.w_in = self._put(torch.cat([t["q"], t["f"], t["v"]], 0))
        self.f_bias, self.lower = self._put(t["f.b"]), self._put(t["lower"])
        self.gnorm, self.w_o = self._put(t["norm"]), self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        hd = self.H * self.dim
        self.w_in = self._rand(gen, 2 * hd + self.H * self.vdim, self.width, std=std)
        self.f_bias = torch.zeros(hd, dtype=self.dtype, device=self.device)
        self.lower = torch.linspace(0.0, 0.9, hd, device=self.device).to(self.dtype)
        self.gnorm = torch.ones(self.vdim, dtype=self.dtype, device=self.device)
        self.w_o = self._rand(gen, self.width, self.H * self.vdim, std=std)

    def alloc_state(self, slots: int) -> None:
        self.rec_state = torch.zeros(slots, self.H, self.dim, self.vdim, dtype=torch.float32, device=self.device)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        cu, slot, reset = ctx.seqs
        hd = self.H * self.dim
        p = linear(h, self.w_in)                                          # [T, q | f | v]
        o = ops.hgrn2_scan(p[:, :hd], p[:, hd:2 * hd], p[:, 2 * hd:], self.f_bias, self.lower, self.gnorm,
                           self.rec_state, cu, slot, reset, self.H, self.dim, self.vdim, self.eps)
        return linear(o, self.w_o)


class PolyNormMLP(_Block):
    """W_down act(W_up h) with act(z) = a N(z) + b N(z^2) + c N(z^3) + e (element-wise powers, N =
    division by the row's root mean square).  Checkpoint tensors ``up down act`` (act = a, b, c, e)."""

    def __init__(self, width: int, ff: int, eps: float, device, dtype):
        super().__init__(device, dtype)
        self.width, self.ff, self.eps = width, ff, float(eps)
        self.w_up = self.w_d = self.coef = None

    def load(self, t: dict) -> None:
        self.w_up, self.w_d, self.coef = self._put(t["up"]), self._put(t["down"]), self._put(t["act"], torch.float32)

    def init_random(self, gen, std: float) -> None:
        self.w_up, self.w_d = self._rand(gen, self.ff, self.width, std=std), self._rand(gen, self.width, self.ff,
                                                                                        std=std)
        self.coef = torch.tensor([1.0, 0.5, 0.25, 0.0], dtype=torch.float32, device=self.device)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return linear(ops.polynorm(linear(h, self.w_up), self.coef, self.eps), self.w_d)


class InputScaledMoE(_Block):
    """Mixture of SwiGLU experts (no biases): router scores s = sigmoid(W_r h) from fp32 logits, the
    ``top`` largest chosen, weights = those scores (not renormalised) applied to the expert's INPUT:
    y = sum_e expert_e(s_e h) (+ shared(h), an always-on expert of its own width).  Checkpoint
    tensors ``router e<j>.gate|up|down [shared.gate|up|down]``.

    Two paths: rows pre-scaled and expanded (``ops.scale_rows``), sorted by expert, through the
    grouped MFMA GEMMs (bf16, widths that are multiples of 32); otherwise every expert over all
    rows as batched library GEMMs with the unchosen rows' inputs zeroed (an expert without biases
    maps 0 to 0, so they add nothing) -- any shape, any dtype, no host synchronisation either way."""

    def __init__(self, width: int, experts: int, top: int, ff: int, shared_ff: int, device, dtype):
        super().__init__(device, dtype)
        self.width, self.E, self.k, self.ff, self.sff = width, experts, top, ff, int(shared_ff or 0)
        self.w_router = self.w13 = self.w2 = self.w_sgu = self.w_sd = None

    def load(self, t: dict) -> None:
        self.w_router = self._put(t["router"])
        self.w13 = self._put(torch.stack([torch.cat([t[f"e{e}.gate"], t[f"e{e}.up"]], 0) for e in range(self.E)]))
        self.w2 = self._put(torch.stack([t[f"e{e}.down"] for e in range(self.E)]))
        if self.sff:
            self.w_sgu, self.w_sd = self._put(torch.cat([t["shared.gate"], t["shared.up"]], 0)), self._put(t["shared.down"])

    def init_random(self, gen, std: float) -> None:
        self.w_router = self._rand(gen, self.E, self.width, std=std)
        self.w13, self.w2 = self._rand(gen, self.E, 2 * self.ff, self.width, std=std), self._rand(
            gen, self.E, self.width, self.ff, std=std)
        if self.sff:
            self.w_sgu, self.w_sd = self._rand(gen, 2 * self.sff, self.width, std=std), self._rand(
                gen, self.width, self.sff, std=std)

    def grouped_ok(self, h: torch.Tensor) -> bool:
        return h.is_cuda and h.dtype == torch.bfloat16 and self.width % 32 == 0 and self.ff % 32 == 0

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        T, W = h.shape
        logits = ops.lm_head_f32(h, self.w_router)                        # fp32 [T, E]
        tw, tid = ops.moe_route(logits, self.k, False, "sigmoid")
        sh = linear(ops.act_and_mul(linear(h, self.w_sgu), 0), self.w_sd) if self.sff else None
        if self.grouped_ok(h):
            y, inv = ops.moe_experts_sorted(ops.scale_rows(h, tw), tid.view(-1), self.w13, self.w2, 0, self.E)
            ones = torch.ones(T, self.k, dtype=torch.float32, device=h.device)   # (per call: a buffer kept across
            # calls would be pinned into captured decode graphs and could not grow afterwards)
            return ops._combine(y, ones, inv, T, self.k, W, 1.0, sh.contiguous() if sh is not None else None)
        wd = torch.zeros(T, self.E, dtype=torch.float32, device=h.device).scatter_(1, tid.long(), tw)
        xe = (wd.t()[:, :, None] * h.float()[None]).to(h.dtype)           # [E, T, W]: s_e h, or 0
        gu = torch.bmm(xe, self.w13.transpose(1, 2))
        hh = ops.act_and_mul(gu.view(self.E * T, 2 * self.ff), 0).view(self.E, T, self.ff)
        y = torch.bmm(hh, self.w2.transpose(1, 2)).float().sum(0)
        return (y if sh is None else y + sh.float()).to(h.dtype)


class TokenSideInput(_Block):
    """Per-layer token input: e = the layer's ``dim``-wide slice of a second embedding row of the
    token; g = gelu_tanh(W_gate x) * e; y = W_proj g.  The caller adds RMSNorm(y) * ``norm`` to the
    stream.  Checkpoint tensors ``gate proj norm`` (the table is shared by all layers)."""

    def __init__(self, width: int, dim: int, col0: int, device, dtype):
        super().__init__(device, dtype)
        self.width, self.dim, self.col0 = width, dim, col0
        self.w_gate = self.w_proj = self.norm = None

    def load(self, t: dict) -> None:
        self.w_gate, self.w_proj, self.norm = self._put(t["gate"]), self._put(t["proj"]), self._put(t["norm"])

    def init_random(self, gen, std: float) -> None:
        self.w_gate, self.w_proj = self._rand(gen, self.dim, self.width, std=std), self._rand(gen, self.width, self.dim,
                                                                                              std=std)
        self.norm = torch.ones(self.width, dtype=self.dtype, device=self.device)

    def forward(self, h: torch.Tensor, ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
        return linear(ops.gelu_gather_mul(linear(h, self.w_gate), ids, table, self.col0), self.w_proj)


def attention_rows(meta: AttnMeta, T: int) -> list:
    """The step's rows for kernels that take one (block-table row, position) per query row:
    segments (first row, end row, block table, block-table row per token, position per token) --
    one for the prompt chunks, one for the single decode rows of a mixed step."""
    return [(s, e, bt, rows, lens - 1) for s, e, bt, rows, lens in latent_rows(meta, T)]


class ConvRotaryAttention(_Block):
    """Grouped-query attention whose q, k and v each pass a short causal depthwise convolution
    (``conv`` taps, no bias, no activation; 0: none) right after the projection; q and k are then
    rotated on the first ``rot_dims`` dims of every head (interleaved or half-split pairs) and,
    after the rotation, divided by their root mean square per head (no weight); score = q.k *
    ``scale``; query i sees keys j with 0 <= i - j < ``window``; softmax whose denominator also
    holds exp(``sink``_h); W_o.  Checkpoint tensors ``q k v [q.conv k.conv v.conv] sink o``;
    state: the last conv - 1 projected rows per request slot."""

    def __init__(self, layer: int, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                 conv: int, rot_base: float, rot_dims: int, scale: float, eps: float, max_positions: int, device,
                 dtype, interleaved: bool = True, unit_norm: bool = True):
        super().__init__(device, dtype)
        if heads % kv_heads or heads // kv_heads > 16:
            raise ValueError(f"attention: {heads} query heads over {kv_heads} kv heads (groups of <= 16 supported)")
        self.layer, self.width, self.Hq, self.Hkv, self.dim, self.vdim = layer, width, heads, kv_heads, dim, vdim
        self.window, self.K = int(window) if window and window > 0 else -1, int(conv or 0)
        self.rot_dims, self.scale, self.eps = int(rot_dims), float(scale), float(eps)
        self.interleaved, self.unit_norm = interleaved, unit_norm
        self.D = attn_tile_dim(max(dim, vdim))
        self.cos_sin = plain_rope_table(rot_base, self.rot_dims, max_positions, self.device) if rot_dims else \
            torch.zeros(max_positions, 0, device=self.device)
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.w_in = self.cq = self.ck = self.cv = self.sink = self.w_o = None
        self.tail = None

    def load(self, t: dict) -> None:
        self.w_in = self._put(torch.cat([t["q"], t["k"], t["v"]], 0))
        if self.K:
            self.cq, self.ck, self.cv = self._put(t["q.conv"]), self._put(t["k.conv"]), self._put(t["v.conv"])
            for n, c, w in (("q", self.nq, self.cq), ("k", self.nk, self.ck), ("v", self.nv, self.cv)):
                if tuple(w.shape) != (c, self.K):
                    raise ValueError(f"{n}.conv: shape {tuple(w.shape)} != [{c}, {self.K}]")
        self.sink, self.w_o = self._put(t["sink"], torch.float32), self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        self.w_in = self._rand(gen, self.nq + self.nk + self.nv, self.width, std=std)
        if self.K:
            self.cq, self.ck, self.cv = (self._rand(gen, c, self.K, std=0.5) for c in (self.nq, self.nk, self.nv))
        self.sink = torch.zeros(self.Hq, dtype=torch.float32, device=self.device)
        self.w_o = self._rand(gen, self.width, self.Hq * self.vdim, std=std)

    def alloc_state(self, slots: int) -> None:
        if self.K > 1:
            self.tail = torch.zeros(slots, self.K - 1, self.nq + self.nk + self.nv, dtype=self.dtype, device=self.device)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        T = h.shape[0]
        nq, nk = self.nq, self.nk
        p = linear(h, self.w_in)                                   # [T, q | k | v]
        q = torch.empty(T, self.Hq, self.D, dtype=h.dtype, device=h.device)
        k_cache, v_cache = ctx.kv.layer(self.layer)
        rows = ctx.cache.get("rows")
        if rows is None and h.is_cuda:
            rows = ctx.cache["rows"] = ops.seq_rows(ctx.seqs, T)
        ops.conv_rope_cache(p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:], self.cq, self.ck, self.cv, self.tail, ctx.seqs,
                            ctx.meta.positions, self.cos_sin, self.rot_dims, self.interleaved, self.unit_norm, self.eps,
                            q, k_cache, v_cache, ctx.meta.slots, self.Hq, self.Hkv, self.dim, self.vdim, rows=rows)
        a = paged_attention(q, k_cache, v_cache, ctx.meta, self.scale, self.window, 0, self.sink)
        if self.D != self.vdim:
            a = a[:, :, :self.vdim].reshape(T, self.Hq * self.vdim)
        return linear(a.view(T, self.Hq * self.vdim), self.w_o)


class TalkingHeadsAttention(_Block):
    """Grouped-query attention without rotation: score = q.k * ``scale`` - r1_h ln(1 + r2_h (i -
    j)) (a per-head logarithmic distance bias); query i sees keys j with 0 <= i - j < ``window``;
    softmax whose denominator also holds exp(``sink``_h); the normalised weights are mixed across
    heads (w_h <- sum_g talk[h, g] w_g) before head h applies them to the values of its own kv
    head; every head's output is multiplied by sigmoid(W_g x)_h; W_o.  Checkpoint tensors ``q k v
    r1 r2 talk sink g o``."""

    def __init__(self, layer: int, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                 scale: float, device, dtype):
        super().__init__(device, dtype)
        if heads % kv_heads or heads // kv_heads > 16:
            raise ValueError(f"attention: {heads} query heads over {kv_heads} kv heads (groups of <= 16 supported)")
        if heads * vdim > 8192:
            raise ValueError(f"talking-heads attention: {heads} heads x {vdim} value dims exceed 8192 outputs per row")
        self.layer, self.width, self.Hq, self.Hkv, self.dim, self.vdim = layer, width, heads, kv_heads, dim, vdim
        self.window, self.scale = int(window) if window and window > 0 else -1, float(scale)
        self.D = attn_tile_dim(max(dim, vdim))
        self.nq, self.nk, self.nv = heads * dim, kv_heads * dim, kv_heads * vdim
        self.w_in = self.r1 = self.r2 = self.talk = self.sink = self.w_o = None
        self._none = torch.zeros(1, 0, device=self.device)

    def load(self, t: dict) -> None:
        f32 = torch.float32
        self.w_in = self._put(torch.cat([t["q"], t["k"], t["v"], t["g"]], 0))
        self.r1, self.r2, self.talk = self._put(t["r1"], f32), self._put(t["r2"], f32), self._put(t["talk"], f32)
        self.sink, self.w_o = self._put(t["sink"], f32), self._put(t["o"])
        if tuple(self.talk.shape) != (self.Hq, self.Hq):
            raise ValueError(f"talk: shape {tuple(self.talk.shape)} != [{self.Hq}, {self.Hq}]")

    def init_random(self, gen, std: float) -> None:
        f32 = dict(dtype=torch.float32, device=self.device)
        H = self.Hq
        self.w_in = self._rand(gen, self.nq + self.nk + self.nv + H, self.width, std=std)
        self.r1, self.r2 = torch.linspace(0.1, 1.0, H, **f32), torch.linspace(0.5, 2.0, H, **f32)
        self.talk = torch.eye(H, **f32) + 0.1 * torch.randn(H, H, generator=gen, **f32)
        self.sink = torch.zeros(H, **f32)
        self.w_o = self._rand(gen, self.width, H * self.vdim, std=std)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        T = h.shape[0]
        nq, nk, nv = self.nq, self.nk, self.nv
        p = linear(h, self.w_in)                                   # [T, q | k | v | gate]
        q = torch.empty(T, self.Hq, self.D, dtype=h.dtype, device=h.device)
        k_cache, v_cache = ctx.kv.layer(self.layer)
        ops.wide_norm_rope_cache(p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:nq + nk + nv], ctx.meta.positions,
                                 self._none, 0, True, None, None, 0.0, q, k_cache, v_cache, ctx.meta.slots, self.Hq,
                                 self.Hkv, self.dim, self.vdim)
        o = torch.empty(T, self.Hq * self.vdim, dtype=h.dtype, device=h.device)
        gate = p[:, nq + nk + nv:]
        meta = ctx.meta
        args = (self.scale, self.window, self.sink, self.r1, self.r2, self.talk)
        if ops.talking_prefill_ok(q, self.Hq, self.D, k_cache.shape[2]):   # bf16: the MFMA kernels
            n = 0 if meta.is_decode else (meta.num_prefill if meta.mode == "mixed" else T)
            if n:                              # prompt chunks: 16 rows x all heads per workgroup
                ops.talking_prefill(q[:n], k_cache, v_cache, meta.block_tables, meta.cu_q, meta.kv_lens, meta.items,
                                    *args, gate[:n], self.vdim, out=o[:n])
            if n < T:                          # single rows: the keys of a row split over workgroups
                bt = meta.block_tables if meta.is_decode else meta.dec_block_tables
                ops.talking_decode(q[n:], k_cache, v_cache, bt, meta.seq_lens, *args, gate[n:], self.vdim, out=o[n:])
        else:                                  # fp32 models, shapes without an MFMA kernel, the CPU: the row kernel
            for s, e, bt, rows, pos in attention_rows(meta, T):
                ops.talking_attn(q[s:e], k_cache, v_cache, bt, rows, pos, *args, gate[s:e], self.vdim, out=o[s:e])
        return linear(o, self.w_o)


class GeluMLP(_Block):
    """W_down gelu(W_up h) with the exact (erf) GELU.  Checkpoint tensors ``up down``."""

    def __init__(self, width: int, ff: int, device, dtype):
        super().__init__(device, dtype)
        self.width, self.ff = width, ff
        self.w_up = self.w_d = None

    def load(self, t: dict) -> None:
        self.w_up, self.w_d = self._put(t["up"]), self._put(t["down"])

    def init_random(self, gen, std: float) -> None:
        self.w_up, self.w_d = self._rand(gen, self.ff, self.width, std=std), self._rand(gen, self.width, self.ff,
                                                                                        std=std)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return linear(ops.act(linear(h, self.w_up).contiguous(), 3), self.w_d)


class GroupRoutedMoE(_Block):
    """Mixture of clamped-GLU experts (:class:`ClampedGLU`'s form, no biases).  Router scores s =
    softmax(W_r h) over all experts from fp32 logits; the choice is made on s + ``correction``,
    among the experts of the ``keep`` best of ``groups`` equal groups of neighbours (a group scores
    by its best choice score; experts of the other groups are excluded outright); the ``top``
    chosen experts' outputs are weighted by their plain scores s (not renormalised).  An optional
    shared expert (own width and ``limit``) runs for every token, times sigmoid(w_sg . h).
    ``act``: the experts' gated activation (2 clamped GLU, 0 plain SiLU GLU: no ``limit``);
    ``renorm``: the chosen scores are divided by their sum (= a softmax over the chosen logits
    alone); ``router_bias``: the router has a bias ``router.b`` that is part of the logits;
    ``correction`` False: no choice-only correction tensor.
    Checkpoint tensors ``router [router.b] [correction] e<j>.gate|up|down [shared.gate|up|down|sg]``.

    The router and the shared gate are one fp32-result GEMM (``[W_r; w_sg]``).  Experts run on the
    grouped MFMA GEMMs (bf16, widths in multiples of 32), otherwise densely: every expert over all
    rows as batched library GEMMs, weighted by the scattered scores (0 for unchosen experts) -- any
    shape, fp32 models; no host synchronisation either way."""

    def __init__(self, width: int, experts: int, top: int, ff: int, limit: float, groups: int, keep: int,
                 shared_ff: int, shared_limit: float, device, dtype, act: int = 2, renorm: bool = False,
                 router_bias: bool = False, correction: bool = True):
        super().__init__(device, dtype)
        if groups < 1 or experts % groups or not 1 <= keep <= groups or top > keep * (experts // groups):
            raise ValueError(f"moe: {experts} experts in {groups} groups, {keep} kept, top {top}")
        if experts > 512 or top > 16:
            raise ValueError(f"moe: {experts} experts / top {top} exceed the router kernel (512 / 16)")
        self.act, self.renorm, self.has_rb, self.has_corr = int(act), bool(renorm), bool(router_bias), bool(correction)
        self.router_b = None
        self.width, self.E, self.k, self.ff, self.limit = width, experts, top, ff, float(limit)
        self.groups, self.keep = groups, keep
        self.sff, self.slimit = int(shared_ff or 0), float(shared_limit or 0.0)
        self.w_router = self.correction = self.w13 = self.w2 = self.w_sgu = self.w_sd = None

    def load(self, t: dict) -> None:
        self.w_router = self._put(torch.cat([t["router"], t["shared.sg"].reshape(1, -1)], 0) if self.sff
                                  else t["router"])
        self.correction = self._put(t["correction"], torch.float32) if self.has_corr else None
        self.router_b = self._put(t["router.b"], torch.float32) if self.has_rb else None
        self.w13 = self._put(torch.stack([torch.cat([t[f"e{e}.gate"], t[f"e{e}.up"]], 0) for e in range(self.E)]))
        self.w2 = self._put(torch.stack([t[f"e{e}.down"] for e in range(self.E)]))
        if self.sff:
            self.w_sgu, self.w_sd = self._put(torch.cat([t["shared.gate"], t["shared.up"]], 0)), self._put(t["shared.down"])

    def init_random(self, gen, std: float) -> None:
        self.w_router = self._rand(gen, self.E + (1 if self.sff else 0), self.width, std=std)
        self.correction = torch.zeros(self.E, dtype=torch.float32, device=self.device) if self.has_corr else None
        self.router_b = torch.zeros(self.E, dtype=torch.float32, device=self.device) if self.has_rb else None
        self.w13, self.w2 = self._rand(gen, self.E, 2 * self.ff, self.width, std=std), self._rand(
            gen, self.E, self.width, self.ff, std=std)
        if self.sff:
            self.w_sgu, self.w_sd = self._rand(gen, 2 * self.sff, self.width, std=std), self._rand(
                gen, self.width, self.sff, std=std)

    def grouped_ok(self, h: torch.Tensor) -> bool:
        return h.is_cuda and h.dtype == torch.bfloat16 and self.width % 32 == 0 and self.ff % 32 == 0

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        T, W = h.shape
        logits = ops.lm_head_f32(h, self.w_router)                        # fp32 [T, E (+ shared gate)]
        tw, tid = ops.moe_route(logits[:, :self.E], self.k, self.renorm, "softmax", bias=self.correction,
                                n_group=self.groups, topk_group=self.keep, group_mode=3 if self.groups > 1 else 0,
                                logit_bias=self.router_b)
        sh = None
        if self.sff:
            a = ops.act_and_mul(linear(h, self.w_sgu).contiguous(), self.act, limit=self.slimit,
                                row_gate=logits[:, self.E])
            sh = linear(a, self.w_sd)
        if self.grouped_ok(h):
            return ops.fused_moe(h, tw, tid, self.w13, self.w2, act=self.act, limit=self.limit,
                                 add=sh.contiguous() if sh is not None else None)
        wd = torch.zeros(T, self.E, dtype=torch.float32, device=h.device).scatter_(1, tid.long(), tw)
        gu = torch.matmul(h, self.w13.transpose(1, 2))                    # [E, T, 2 ff]
        hh = ops.act_and_mul(gu.view(self.E * T, 2 * self.ff), self.act, limit=self.limit).view(self.E, T, self.ff)
        y = (torch.bmm(hh, self.w2.transpose(1, 2)).float() * wd.t()[:, :, None]).sum(0)
        return (y if sh is None else y + sh.float()).to(h.dtype)


class KeyValuedAttention(_Block):
    """Grouped-query attention without a value projection: q = W_q h, k = W_k h, and the values
    are the keys as projected (v = k BEFORE the rotation).  q and k are rotated on the first
    ``rot_dims`` dims of every head (half-split pairs i / i + rot_dims/2 by default, or
    ``interleaved`` neighbours); score = q.k * ``scale`` * temp_h (a learned per-head temperature);
    query i sees keys j with 0 <= i - j < ``window``; softmax whose denominator also holds
    exp(``sink``_h) (not scaled, not multiplied by the temperature); W_o on the concatenated heads.
    Checkpoint tensors ``q k temp sink o``.  The temperature is folded into the rotated query in
    fp32 before its one rounding (``ops.wide_norm_rope_cache(q_scale=)``), the key projection is
    written into the paged cache twice: rotated as the key row, unrotated as the value column."""

    def __init__(self, layer: int, width: int, heads: int, kv_heads: int, dim: int, window: int, rot_base: float,
                 rot_dims: int, scale: float, max_positions: int, device, dtype, interleaved: bool = False):
        super().__init__(device, dtype)
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} query heads do not divide over {kv_heads} kv heads")
        self.layer, self.width, self.Hq, self.Hkv, self.dim = layer, width, heads, kv_heads, dim
        self.window = int(window) if window and window > 0 else -1
        self.rot_dims, self.scale, self.interleaved = int(rot_dims), float(scale), bool(interleaved)
        self.D = attn_tile_dim(dim)
        self.cos_sin = plain_rope_table(rot_base, self.rot_dims, max_positions, self.device) if rot_dims else \
            torch.zeros(max_positions, 0, device=self.device)
        self.nq, self.nk = heads * dim, kv_heads * dim
        self.w_in = self.temp = self.sink = self.w_o = None

    def load(self, t: dict) -> None:
        self.w_in = self._put(torch.cat([t["q"], t["k"]], 0))
        self.temp, self.sink = self._put(t["temp"], torch.float32), self._put(t["sink"], torch.float32)
        self.w_o = self._put(t["o"])
        if tuple(self.w_in.shape) != (self.nq + self.nk, self.width) or self.temp.numel() != self.Hq:
            raise ValueError(f"attention: q / k {tuple(self.w_in.shape)} or temp {tuple(self.temp.shape)} do not fit "
                             f"{self.Hq} + {self.Hkv} heads of {self.dim}")

    def init_random(self, gen, std: float) -> None:
        self.w_in = self._rand(gen, self.nq + self.nk, self.width, std=std)
        self.temp = torch.linspace(0.75, 1.25, self.Hq, dtype=torch.float32, device=self.device)
        self.sink = torch.zeros(self.Hq, dtype=torch.float32, device=self.device)
        self.w_o = self._rand(gen, self.width, self.nq, std=std)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        T, nq = h.shape[0], self.nq
        p = linear(h, self.w_in)                                   # [T, q | k]
        q = torch.empty(T, self.Hq, self.D, dtype=h.dtype, device=h.device)
        k_cache, v_cache = ctx.kv.layer(self.layer)
        ops.wide_norm_rope_cache(p[:, :nq], p[:, nq:], p[:, nq:], ctx.meta.positions, self.cos_sin, self.rot_dims,
                                 self.interleaved, None, None, 0.0, q, k_cache, v_cache, ctx.meta.slots, self.Hq,
                                 self.Hkv, self.dim, self.dim, q_scale=self.temp)
        a = paged_attention(q, k_cache, v_cache, ctx.meta, self.scale, self.window, 0, self.sink)
        if self.D != self.dim:
            a = a[:, :, :self.dim].reshape(T, nq)
        return linear(a.view(T, nq), self.w_o)


class DifferentialAttention(_Block):
    """Differential attention.  q = W_q h has ``heads`` x 2 x ``dim`` rows and k = W_k h ``kv_heads``
    x 2 x ``dim``, head by head as [map 1, map 2]; v = W_v h has ``kv_heads`` x ``vdim``.  Every map is
    rotated on its first ``rot_dims`` dims (interleaved pairs by default) and is a windowed softmax
    attention of its own (score = q.k * ``scale``, 0 <= i - j < ``window``) over the head's values;
    with lam = exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff`` (one number per layer): o = a1 - lam a2,
    o / sqrt(mean(o^2) + eps) over ``vdim`` (no weight), times (1 - ``diff``); W_o.  Checkpoint
    tensors ``q k v lq1 lk1 lq2 lk2 o``.

    The maps run as separate heads of the framework's paged attention kernels: 2 x ``heads`` query
    heads over 2 x ``kv_heads`` key heads.  The rows of W_q are reordered at load to [kv group][map]
    [head of the group], so that query head (g, m, r) reads key head 2 g + m, which is where k's
    layout already has it; the cache holds the group's values under both key heads (``v_rep`` =
    2).  ``ops.diff_head_norm`` then combines the two outputs of a head, norms and rounds once."""

    def __init__(self, layer: int, width: int, heads: int, kv_heads: int, dim: int, vdim: int, window: int,
                 rot_base: float, rot_dims: int, scale: float, diff: float, eps: float, max_positions: int, device,
                 dtype, interleaved: bool = True):
        super().__init__(device, dtype)
        if heads % kv_heads:
            raise ValueError(f"attention: {heads} query heads do not divide over {kv_heads} kv heads")
        self.layer, self.width, self.H, self.G, self.dim, self.vdim = layer, width, heads, kv_heads, dim, vdim
        self.Hq, self.Hkv, self.group = 2 * heads, 2 * kv_heads, heads // kv_heads
        self.window = int(window) if window and window > 0 else -1
        self.rot_dims, self.scale, self.diff, self.eps = int(rot_dims), float(scale), float(diff), float(eps)
        self.interleaved = bool(interleaved)
        self.D = attn_tile_dim(max(dim, vdim))
        self.cos_sin = plain_rope_table(rot_base, self.rot_dims, max_positions, self.device) if rot_dims else \
            torch.zeros(max_positions, 0, device=self.device)
        self.nq, self.nk, self.nv = 2 * heads * dim, 2 * kv_heads * dim, kv_heads * vdim
        self.lam = float(diff)
        self.w_in = self.w_o = None

    def load(self, t: dict) -> None:
        G, R, d = self.G, self.group, self.dim
        wq = t["q"]
        if tuple(wq.shape) != (self.nq, self.width):
            raise ValueError(f"attention_2: q {tuple(wq.shape)} != [{self.nq}, {self.width}]")
        wq = wq.view(G, R, 2, d, self.width).permute(0, 2, 1, 3, 4).reshape(self.nq, self.width)
        self.w_in = self._put(torch.cat([wq, t["k"], t["v"]], 0))
        f = lambda n: t[n].double()   # noqa: E731
        self.lam = math.exp(float((f("lq1") * f("lk1")).sum())) - math.exp(float((f("lq2") * f("lk2")).sum())) + self.diff
        self.w_o = self._put(t["o"])

    def init_random(self, gen, std: float) -> None:
        self.w_in = self._rand(gen, self.nq + self.nk + self.nv, self.width, std=std)
        self.lam = self.diff
        self.w_o = self._rand(gen, self.width, self.H * self.vdim, std=std)

    def forward(self, h: torch.Tensor, ctx: MixerCtx) -> torch.Tensor:
        T, nq, nk = h.shape[0], self.nq, self.nk
        p = linear(h, self.w_in)                                   # [T, q (group, map, head) | k | v]
        q = torch.empty(T, self.Hq, self.D, dtype=h.dtype, device=h.device)
        k_cache, v_cache = ctx.kv.layer(self.layer)
        ops.wide_norm_rope_cache(p[:, :nq], p[:, nq:nq + nk], p[:, nq + nk:], ctx.meta.positions, self.cos_sin,
                                 self.rot_dims, self.interleaved, None, None, 0.0, q, k_cache, v_cache, ctx.meta.slots,
                                 self.Hq, self.Hkv, self.dim, self.vdim, v_rep=2)
        a = paged_attention(q, k_cache, v_cache, ctx.meta, self.scale, self.window)
        o = ops.diff_head_norm(a, self.lam, self.eps, 1.0 - self.diff, self.group, self.vdim)
        return linear(o, self.w_o)
