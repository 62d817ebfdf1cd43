"""Slow fp64 implementation of the Nivasun design, one function per mechanism, written from the
equations alone (no code shared with ``ome_amd``), plus makers of small random configs and
checkpoints for the tests.  Everything works on one whole sequence at a time."""
from __future__ import annotations

import json
import math
import os

import torch

F64 = torch.float64


# ------------------------------------------------------------------------------------ pieces
def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def sigmoid(x):
    return 1 / (1 + torch.exp(-x))


def silu(x):
    return x * sigmoid(x)


def hashed_rows(tokens, b):
    """Row of the pair table for every token: (previous * mul_prev + token * mul_cur) mod buckets,
    the extra last row for a sequence's first token."""
    rows = [b["buckets"]]
    for prev, cur in zip(tokens[:-1], tokens[1:]):
        rows.append((prev * b["mul_prev"] + cur * b["mul_cur"]) % b["buckets"])
    return rows


def embed_tokens(tokens, w, e):
    x = w["embed"][tokens] * e["scale"]
    if e.get("bigram"):
        x = x + w["bigram"][hashed_rows(tokens, e["bigram"])]
    return x


def causal_conv(u, w):
    """y_t = sum_j w[:, j] u_{t - K + 1 + j}, rows before the start are zero; u [T, C], w [C, K]."""
    T, K = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for j in range(K):
        back = K - 1 - j                      # tap j reads the row `back` steps before
        if back < T:
            y[back:] += w[:, j] * u[:T - back]
    return y


def angles(T, dims, base):
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    a = torch.arange(T, dtype=F64)[:, None] * f[None]
    return torch.cos(a)[:, None], torch.sin(a)[:, None]


def rotate_halves(x, dims, base):
    """x [T, H, d]: dim i pairs with dim i + dims/2 (i < dims/2) and turns by t * base^(-2i/dims)."""
    if not dims:
        return x
    c, s = angles(x.shape[0], dims, base)
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    out = x.clone()
    out[..., :dims // 2] = u * c - v * s
    out[..., dims // 2:dims] = v * c + u * s
    return out


def rotate_neighbours(x, dims, base):
    """x [T, H, d]: dims (2i, 2i+1), i < dims/2, turn by t * base^(-2i/dims); the rest passes."""
    if not dims:
        return x
    c, s = angles(x.shape[0], dims, base)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def window_mask(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None]
    return (j <= i) & (i - j < size)


def masked_softmax(score, visible, sink=None):
    """score [H, T, T] -> weights; ``sink`` [H] only enlarges the denominator."""
    s = score.masked_fill(~visible[None], -math.inf)
    m = s.max(-1).values
    if sink is not None:
        m = torch.maximum(m, sink[:, None])
    e = torch.exp(s - m[..., None])
    den = e.sum(-1)
    if sink is not None:
        den = den + torch.exp(sink[:, None] - m)
    return e / den[..., None]


def key_valued_attention(h, w, m):
    """Grouped-query attention whose values are the unrotated keys; per-head temperature and sink."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    rot = m.get("rot") or {}
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v = k
    q, k = rotate_halves(q, rot.get("dims", 0), rot.get("base", 1.0)), rotate_halves(k, rot.get("dims", 0), rot.get("base", 1.0))
    kk, vv = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    score = torch.einsum("ihd,jhd->hij", q, kk) * m["scale"] * w["temp"][:, None, None]
    p = masked_softmax(score, window_mask(T, m["mask"]["size"]), w["sink"])
    o = torch.einsum("hij,jhd->ihd", p, vv).reshape(T, H * d)
    return o @ w["o"].T


def latent_attention(h, w, m, eps):
    """Queries and keys / values through normed low-rank latents, no positions, gated output."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    cq = rms_unit(h @ w["dq"].T, eps) * w["dq.norm"]
    q = (cq @ w["uq"].T).view(T, H, d)
    c = rms_unit(h @ w["dkv"].T, eps) * w["dkv.norm"]
    k = (c @ w["uk"].T).view(T, H, d)
    v = (c @ w["uv"].T).view(T, H, dv)
    score = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    p = masked_softmax(score, window_mask(T, m["mask"]["size"]))
    o = torch.einsum("hij,jhd->ihd", p, v).reshape(T, H * dv)
    return (o * sigmoid(h @ w["g"].T)) @ w["o"].T


def difference_lambda(w, diff):
    return math.exp(float((w["lq1"] * w["lk1"]).sum())) - math.exp(float((w["lq2"] * w["lk2"]).sum())) + diff


def differential_attention(h, w, m, eps):
    """Two softmax maps per head over the same values; the second is taken off the first."""
    T = h.shape[0]
    H, G, d, dv, diff = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["diff"]
    rot = m.get("rot") or {}
    rd, rb = rot.get("dims", 0), rot.get("base", 1.0)
    q = (h @ w["q"].T).view(T, H * 2, d)          # head by head: map 1, map 2
    k = (h @ w["k"].T).view(T, G * 2, d)
    v = (h @ w["v"].T).view(T, G, dv)
    q, k = rotate_neighbours(q, rd, rb).view(T, H, 2, d), rotate_neighbours(k, rd, rb).view(T, G, 2, d)
    kk, vv = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    vis = window_mask(T, m["mask"]["size"])
    outs = []
    for a in range(2):
        score = torch.einsum("ihd,jhd->hij", q[:, :, a], kk[:, :, a]) * m["scale"]
        outs.append(torch.einsum("hij,jhd->ihd", masked_softmax(score, vis), vv))
    o = outs[0] - difference_lambda(w, diff) * outs[1]
    o = rms_unit(o, eps) * (1 - diff)
    return o.reshape(T, H * dv) @ w["o"].T


def glu_expert(h, w, pre):
    return (silu(h @ w[pre + "gate"].T) * (h @ w[pre + "up"].T)) @ w[pre + "down"].T


def router_logits(h, w):
    return h @ w["router"].T + w["router.b"]


def moe_ff(h, w, f):
    """The ``top`` experts by logit, weighted by the softmax over the chosen logits only, plus the
    always-on expert times a per-token sigmoid gate."""
    top = f["router"]["top"]
    z = router_logits(h, w)
    val, idx = z.topk(top, -1)
    p = torch.softmax(val, -1)
    y = torch.zeros_like(h)
    for e in range(f["router"]["experts"]):
        share = (p * (idx == e)).sum(-1, keepdim=True)        # the token's weight for expert e, 0 if not chosen
        rows = share[:, 0] > 0
        if rows.any():
            y[rows] += share[rows] * glu_expert(h[rows], w, f"e{e}.")
    if f.get("shared"):
        y = y + glu_expert(h, w, "shared.") * sigmoid(h @ w["shared.sg"].T)
    return y


def sub(w, prefix):
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def run_order(cfg):
    """(layer, pass, first layer of a pass?) in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, 0, False) for i in range(n)]
    a, b, times = lp["start"], lp["stop"], lp["times"]
    return [(i, 0, False) for i in range(a)] + [(i, p, i == a) for p in range(times) for i in range(a, b)] + \
        [(i, 0, False) for i in range(b, n)]


def forward(cfg, weights, tokens, residuals=None, margins=None):
    """Logits [T, vocab] (fp64) of one whole sequence; ``residuals``: a list that receives the
    stream after every layer run; ``margins``: a one-element list that receives the smallest gap
    between the last chosen and the first unchosen router logit."""
    W64 = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = embed_tokens(list(tokens), W64, cfg["embedding"])
    for i, p, first in run_order(cfg):
        L = cfg["layers"][i]
        w = sub(W64, f"l{i}.")
        if first:
            x = x + W64["loop.step"][p]
        h = rms_unit(x, eps) * w["norm1"]
        taps = (cfg.get("canon") or {}).get("taps", 0)
        hm = h + causal_conv(h, w["canon1"]) if taps else h
        mw, m = sub(w, "mix."), L["mixer"]
        if L["type"] == "attention":
            y = key_valued_attention(hm, mw, m)
        elif L["type"] == "latent_attention":
            y = latent_attention(hm, mw, m, eps)
        elif L["type"] == "attention_2":
            y = differential_attention(hm, mw, m, eps)
        else:
            raise ValueError(L["type"])
        f = L.get("mlp")
        if f:
            fw = sub(w, "mlp.")
            if margins is not None and f["router"]["top"] < f["router"]["experts"]:
                srt = router_logits(h, fw).sort(-1, descending=True).values
                t = f["router"]["top"]
                margins[0] = min(margins[0], float((srt[:, t - 1] - srt[:, t]).min()))
            y = y + moe_ff(h, fw, f)
        x = x + y
        if residuals is not None:
            residuals.append(x.clone())
    z = (rms_unit(x, eps) * W64["final.norm"]) @ W64["head"].T
    cap = cfg.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z


# ------------------------------------------------------------------------------------ makers
def moe(experts=5, top=2, ff=12, shared_ff=10):
    f = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff}
    return f


def keyed_layer(heads=4, kv_heads=2, dim=8, window=7, rot_dims=4, base=100.0, scale=0.5, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": window}, "scale": scale,
         "rot": {"base": base, "dims": rot_dims}}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent_layer(heads=3, dim=8, vdim=6, kv_rank=10, q_rank=12, window=9, scale=0.4, mlp=None):
    m = {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank, "q_rank": q_rank, "mask": {"size": window},
         "scale": scale}
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def diff_layer(heads=4, kv_heads=2, dim=6, vdim=10, window=8, rot_dims=4, base=50.0, scale=0.6, diff=0.3, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale,
         "diff": diff, "rot": {"base": base, "dims": rot_dims}}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def make_config(layers, width=24, vocab=41, eps=1e-5, loop=None, taps=3, emb_scale=3.0, buckets=13, mul_prev=5,
                mul_cur=3, softcap=20.0):
    cfg = {"architecture": "Nivasun", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width,
           "canon": {"taps": taps}, "logit_softcap": softcap,
           "embedding": {"scale": emb_scale, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, dtype=torch.bfloat16):
    """Random checkpoint tensors (values exactly representable in ``dtype``), sized so that the
    stream stays O(1) and scores spread over a few units."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(dtype)

    def lin(o, i, gain=1.0):
        return rnd(o, i, s=gain / math.sqrt(i))

    def one():
        return (1.0 + 0.2 * torch.randn((), generator=g)).to(dtype)

    e = cfg["embedding"]
    t = {"embed": rnd(V, W, s=1.0 / e["scale"]), "final.norm": one(), "head": lin(V, W, 2.0)}
    if e.get("bigram"):
        t["bigram"] = rnd(e["bigram"]["buckets"] + 1, W, s=0.5)
    if cfg.get("loop"):
        t["loop.step"] = rnd(cfg["loop"]["times"], W, s=0.3)
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        t[p + "norm1"] = one()
        if taps:
            t[p + "canon1"] = rnd(W, taps, s=0.4)
        if L["type"] == "attention":
            G = m["kv_heads"]
            t[p + "mix.q"], t[p + "mix.k"] = lin(H * d, W, 1.5), lin(G * d, W, 1.5)
            t[p + "mix.temp"] = (0.5 + torch.rand(H, generator=g)).to(dtype)
            t[p + "mix.sink"] = rnd(H)
        elif L["type"] == "attention_2":
            G = m["kv_heads"]
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = lin(2 * H * d, W, 1.5), lin(2 * G * d, W, 1.5), lin(G * dv, W)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                t[p + "mix." + n] = rnd(d, s=0.3)
        else:
            R, Q = m["kv_rank"], m["q_rank"]
            t[p + "mix.dq"], t[p + "mix.dq.norm"], t[p + "mix.uq"] = lin(Q, W), 1 + rnd(Q, s=0.1), lin(H * d, Q, 1.5)
            t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = lin(R, W), 1 + rnd(R, s=0.1)
            t[p + "mix.uk"], t[p + "mix.uv"], t[p + "mix.g"] = lin(H * d, R, 1.5), lin(H * dv, R), lin(H * dv, W)
        t[p + "mix.o"] = lin(W, H * dv, 0.5)
        f = L.get("mlp")
        if not f:
            continue
        E, ff = f["router"]["experts"], f["expert"]["ff"]
        t[p + "mlp.router"], t[p + "mlp.router.b"] = lin(E, W, 2.0), rnd(E, s=0.3)
        for j in range(E):
            t[p + f"mlp.e{j}.gate"], t[p + f"mlp.e{j}.up"] = lin(ff, W), lin(ff, W)
            t[p + f"mlp.e{j}.down"] = lin(W, ff, 0.5)
        sh = f.get("shared")
        if sh:
            t[p + "mlp.shared.gate"], t[p + "mlp.shared.up"] = lin(sh["ff"], W), lin(sh["ff"], W)
            t[p + "mlp.shared.down"], t[p + "mlp.shared.sg"] = lin(W, sh["ff"], 0.5), lin(1, W)
    return t


def write_model(folder, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def router_margin(cfg, weights, tokens):
    """Smallest gap between the last chosen and the first unchosen router logit over all routed
    evaluations of a prompt (infinite when every expert is always chosen)."""
    m = [math.inf]
    forward(cfg, weights, tokens, margins=m)
    return m[0]
