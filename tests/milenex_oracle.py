"""Slow fp64 implementation of the Milenex design, one function per mechanism, written from the
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


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is the offset from one."""
    return rms_unit(x, eps) * (1 + w)


def sigmoid(x):
    return 1 / (1 + torch.exp(-x))


def gelu_erf(z):
    return 0.5 * z * (1 + torch.erf(z / math.sqrt(2.0)))


def token_shift(h, mu):
    """h [T, W]: every row moves towards the row before it (zeros before the first) by mu."""
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)
    return h + (prev - h) * mu


def causal_conv(u, w):
    """y_t = sum_j w[:, j] u_{t - K + 1 + j}, rows before the start are zero; u [T, C], w [C, K]."""
    T, K = u.shape[0], w.shape[1]
    y = torch.zeros_like(u)
    for j in range(K):
        back = K - 1 - j
        if back < T:
            y[back:] += w[:, j] * u[:T - back]
    return y


def rotate_pairs(x, dims, base):
    """x [T, H, d]: dims (2i, 2i+1), i < dims/2, turn by t * base^(-2i/dims); the rest passes."""
    if not dims:
        return x
    T = x.shape[0]
    f = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)
    a = torch.arange(T, dtype=F64)[:, None] * f[None]
    c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def window_mask(T, size):
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None]
    return (j <= i) & (i - j < size)


def sink_softmax(score, visible, sink):
    """score [H, T, T], sink [H] -> weights [H, T, T]; the sink only enlarges the denominator."""
    s = score.masked_fill(~visible[None], -math.inf)
    m = torch.maximum(s.max(-1).values, sink[:, None])
    e = torch.exp(s - m[..., None])
    return e / (e.sum(-1) + torch.exp(sink[:, None] - m))[..., None]


def rotary_attention(h, w, m, eps):
    """The mixer with short convolutions, rotary pairs, unit-RMS q / k, window and sink."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ w["q"].T, h @ w["k"].T, h @ w["v"].T
    if m.get("conv"):
        q, k, v = causal_conv(q, w["q.conv"]), causal_conv(k, w["k.conv"]), causal_conv(v, w["v.conv"])
    rot = m.get("rot") or {}
    q = rotate_pairs(q.view(T, H, d), rot.get("dims", 0), rot.get("base", 1.0))
    k = rotate_pairs(k.view(T, G, d), rot.get("dims", 0), rot.get("base", 1.0))
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    v = v.view(T, G, dv)
    kk, vv = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    score = torch.einsum("ihd,jhd->hij", q, kk) * m["scale"]
    p = sink_softmax(score, window_mask(T, m["mask"]["size"]), w["sink"])
    o = torch.einsum("hij,jhd->ihd", p, vv).reshape(T, H * dv)
    return o @ w["o"].T


def biased_attention(h, w, m):
    """The mixer without rotation: logarithmic distance bias, window, sink, weights mixed across
    heads after the softmax, one output gate per head."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = (h @ w["q"].T).view(T, H, d), (h @ w["k"].T).view(T, G, d), (h @ w["v"].T).view(T, G, dv)
    kk, vv = k.repeat_interleave(H // G, 1), v.repeat_interleave(H // G, 1)
    dist = (torch.arange(T)[:, None] - torch.arange(T)[None]).clamp(min=0).to(F64)
    score = torch.einsum("ihd,jhd->hij", q, kk) * m["scale"]
    score = score - w["r1"][:, None, None] * torch.log(1 + w["r2"][:, None, None] * dist[None])
    p = sink_softmax(score, window_mask(T, m["mask"]["size"]), w["sink"])
    p = torch.einsum("hg,gij->hij", w["talk"], p)
    o = torch.einsum("hij,jhd->ihd", p, vv)
    o = o * sigmoid(h @ w["g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w["o"].T


def dense_ff(h, w):
    return gelu_erf(h @ w["up"].T) @ w["down"].T


def clamped_expert(h, gate, up, down, limit):
    g = (h @ gate.T).clamp(max=limit)
    u = (h @ up.T).clamp(-limit, limit)
    return (g * sigmoid(1.702 * g) * (u + 1)) @ down.T


def route(h, w, r):
    """(scores s [T, E], chosen [T, top]) -- the choice adds the correction and is limited to the
    best groups; the weights are the plain scores."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ w["router"].T, -1)
    c = s + w["correction"]
    g = r.get("groups")
    if g and g["count"] > 1:
        n = g["count"]
        best = c.view(-1, n, E // n).max(-1).values.topk(g["keep"], -1).indices
        ok = torch.zeros(c.shape[0], n, dtype=torch.bool).scatter_(1, best, True).repeat_interleave(E // n, 1)
        c = c.masked_fill(~ok, -math.inf)
    return s, c.topk(top, -1).indices


def moe_ff(h, w, f):
    s, chosen = route(h, w, f["router"])
    y = torch.zeros_like(h)
    lim = f["expert"]["limit"]
    for t in range(h.shape[0]):
        for e in chosen[t].tolist():
            y[t] += s[t, e] * clamped_expert(h[t:t + 1], w[f"e{e}.gate"], w[f"e{e}.up"], w[f"e{e}.down"], lim)[0]
    sh = f.get("shared")
    if sh:
        y = y + sigmoid(h @ w["shared.sg"].T) * clamped_expert(h, w["shared.gate"], w["shared.up"], w["shared.down"],
                                                               sh["limit"])
    return y


def router_margin(cfg, weights, tokens):
    """Smallest gap between the last chosen and the first unchosen choice score over all routed
    evaluations of a prompt (a prompt with a tiny margin is a coin toss for a 16-bit run)."""
    out = [math.inf]
    forward(cfg, weights, tokens, margins=out)
    return out[0]


# ------------------------------------------------------------------------------------ the model
def layer_runs(cfg):
    """[(layer, pass)] in execution order: layers start .. stop-1 repeat ``times`` times."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp or lp.get("times", 1) <= 1:
        return [(i, 0) for i in range(n)]
    a, b = lp["start"], lp["stop"]
    runs = [(i, 0) for i in range(a)]
    for p in range(lp["times"]):
        runs += [(i, p) for i in range(a, b)]
    return runs + [(i, 0) for i in range(b, n)]


def sub(weights, prefix):
    return {k[len(prefix):]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg, weights, tokens, residuals=None, margins=None):
    """tokens (list) -> logits [T, vocab] fp64.  ``residuals``: a list that receives the stream
    after every layer run."""
    W64 = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x0 = W64["embed"][torch.tensor(tokens)]
    x = x0.clone()
    lp = cfg.get("loop") or {}
    for i, p in layer_runs(cfg):
        if p > 0 and i == lp["start"]:
            x = x + x0
        L = cfg["layers"][i]
        w = sub(W64, f"l{i}.")
        h = token_shift(offset_norm(x, w["norm1"], eps), w["shift"])
        if L["type"] == "attention":
            x = x + rotary_attention(h, sub(w, "mix."), L["mixer"], eps)
        elif L["type"] == "attention_2":
            x = x + biased_attention(h, sub(w, "mix."), L["mixer"])
        else:
            raise ValueError(L["type"])
        f = L.get("mlp")
        if f:
            h = offset_norm(x, w["norm2"], eps)
            fw = sub(w, "mlp.")
            if f["kind"] == "dense":
                x = x + dense_ff(h, fw)
            else:
                if margins is not None:
                    s, chosen = route(h, fw, f["router"])
                    c = s + fw["correction"]
                    r = f["router"]
                    if r["top"] < r["experts"]:
                        srt = c.sort(-1, descending=True).values
                        margins[0] = min(margins[0], float((srt[:, r["top"] - 1] - srt[:, r["top"]]).min()))
                x = x + moe_ff(h, fw, f)
        if residuals is not None:
            residuals.append(x.clone())
    return offset_norm(x, W64["final.norm"], eps) @ W64["head"].T


# ------------------------------------------------------------------------------------ makers
def rotary_layer(heads=4, kv_heads=2, dim=8, vdim=6, window=7, conv=3, rot_dims=4, base=100.0, scale=0.5, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale,
         "rot": {"base": base, "dims": rot_dims}}
    if conv:
        m["conv"] = conv
    return {"type": "attention", "mixer": m, "mlp": mlp}


def biased_layer(heads=6, kv_heads=2, dim=6, vdim=10, window=9, scale=0.6, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window}, "scale": scale}
    return {"type": "attention_2", "mixer": m, "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared_ff, groups=1, keep=1, limit=1.25, shared_limit=0.75):
    f = {"kind": "moe", "expert": {"ff": ff, "limit": limit},
         "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    if shared_ff:
        f["shared"] = {"ff": shared_ff, "limit": shared_limit}
    return f


def make_config(layers, width=24, vocab=41, eps=1e-5, loop=None):
    cfg = {"architecture": "Milenex", "layers": layers, "norm": {"eps": eps}, "vocab": vocab, "width": width}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, dtype=torch.bfloat16, std=None):
    """Random checkpoint tensors (values exactly representable in ``dtype``), sized so that the
    stream stays O(1) and scores spread over a few units."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(dtype)

    def lin(o, i, gain=1.0):
        return rnd(o, i, s=gain / math.sqrt(i))

    t = {"embed": rnd(V, W), "final.norm": rnd(W, s=0.1), "head": lin(V, W)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t[p + "norm1"], t[p + "shift"] = rnd(W, s=0.1), torch.rand(W, generator=g).to(dtype)
        t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = lin(H * d, W), lin(G * d, W), lin(G * dv, W)
        t[p + "mix.o"] = lin(W, H * dv, 0.5)
        t[p + "mix.sink"] = rnd(H)
        if L["type"] == "attention":
            if m.get("conv"):
                for n, c in (("q", H * d), ("k", G * d), ("v", G * dv)):
                    t[p + f"mix.{n}.conv"] = rnd(c, m["conv"], s=0.6)
        else:
            t[p + "mix.r1"] = (torch.rand(H, generator=g) * 1.5).to(dtype)
            t[p + "mix.r2"] = (torch.rand(H, generator=g) * 2 + 0.1).to(dtype)
            t[p + "mix.talk"] = (torch.eye(H) + torch.randn(H, H, generator=g) * 0.3).to(dtype)
            t[p + "mix.g"] = lin(H, W)
        f = L.get("mlp")
        if not f:
            continue
        t[p + "norm2"] = rnd(W, s=0.1)
        if f["kind"] == "dense":
            t[p + "mlp.up"], t[p + "mlp.down"] = lin(f["ff"], W), lin(W, f["ff"], 0.5)
            continue
        E, ff = f["router"]["experts"], f["expert"]["ff"]
        t[p + "mlp.router"], t[p + "mlp.correction"] = lin(E, W, 2.0), rnd(E, s=0.1)
        for e in range(E):
            t[p + f"mlp.e{e}.gate"], t[p + f"mlp.e{e}.up"] = lin(ff, W), lin(ff, W)
            t[p + f"mlp.e{e}.down"] = lin(W, ff, 0.5)
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
