"""Layer-list designs beside their closest existing model at equal size (``bench.py --arch-compare
[--arch-design zavilorn|metitar|milenex|nivasun]``).

Nivasun (parallel blocks: one norm feeding a mixer -- differential, key-valued or windowed latent
attention behind a short convolution -- and a biased-router mixture of SiLU-GLU experts with a gated
shared expert, on a hashed token-pair embedding) stands beside the same GPT-OSS-style stack of the
same width, depth, effective head counts, window and expert sizes.

Milenex (token shift, sliding-window attention with sinks: one kind with short convolutions, rotary
pairs and unit-RMS q / k, one with a logarithmic distance bias and weights mixed across heads;
group-routed clamped-GLU experts plus a gated shared expert) stands beside a GPT-OSS-style stack
(sliding-window attention with sinks, clamped-GLU experts) of the same width, depth, heads, window
and expert sizes.

Metitar (latent attention + HGRN2, PolyNorm / input-scaled MoE feed-forwards) stands beside a
DeepSeek-V2-style stack (multi-head latent attention, dense then routed feed-forwards with shared
experts) of the same width, depth, head count, latent width and expert sizes; its kernel table sets
every kernel added for the design next to the like kernel of the existing models.

Zavilorn beside the closest existing hybrid (NemotronH: Mamba-2 + attention + dense MLP) at equal
width, depth and mixer sizes, random weights: engine-level prefill / decode throughput, and a
per-kernel table that sets every kernel added for the design next to the like kernel of the
existing models with its share of the HBM roofline (``bench.py --arch-compare``).

Sizes resemble real layers (width 2048 / 4096, 128-wide heads, Mamba-2 heads of 64 x 128 state).
The Zavilorn stack is [parallel + feed-forward, mamba2, mamba2, mamba2] x 2; the NemotronH stack
``*-MMM*-MMM`` has the same attention, MLP width and Mamba-2 layers (it has no delta-rule mixer,
so its attention blocks are lighter; Qwen3-Next's Gated DeltaNet kernel is the delta rule's like
kernel in the table).
"""
from __future__ import annotations

import json
import time

import torch

HBM_GBS = 8000.0    # MI355X HBM3E peak, GB/s (the roofline of every kernel in the table)

SIZES = {
    "2k": dict(width=2048, heads=16, kv=4, ff=5632, mheads=64, vocab=32768),
    "4k": dict(width=4096, heads=32, kv=8, ff=14336, mheads=128, vocab=32768),
}


def zavilorn_config(s: dict, window: int = 1024, keep_first: int = 8) -> dict:
    par = {"type": "parallel",
           "mixer": {"left": {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128,
                              "mask": {"size": window, "keep_first": keep_first},
                              "rot": {"base": 10000.0, "dims": 64}, "scale": 128 ** -0.5},
                     "right": {"heads": s["heads"], "kv_heads": s["heads"] // 2, "dim": 128, "vdim": 128, "conv": 4},
                     "left_scale": 0.5, "right_scale": 0.5},
           "mlp": {"kind": "dense", "ff": s["ff"], "limit": 7.0}}
    mam = {"type": "mamba2", "mixer": {"heads": s["mheads"], "vdim": 64, "state": 128, "groups": 8, "conv": 4,
                                       "norm_groups": 8}, "mlp": None}
    return {"architecture": "Zavilorn", "embedding": {"scale": 1.0}, "layers": [par, mam, mam, mam] * 2,
            "norm": {"eps": 1e-6}, "vocab": s["vocab"], "width": s["width"], "max_positions": 8192}


def nemotron_config(s: dict) -> dict:
    return dict(architectures=["NemotronHForCausalLM"], model_type="nemotron_h", hidden_size=s["width"],
                hybrid_override_pattern="*-MMM*-MMM", num_attention_heads=s["heads"], num_key_value_heads=s["kv"],
                head_dim=128, intermediate_size=s["ff"], mlp_hidden_act="relu2", mamba_num_heads=s["mheads"],
                mamba_head_dim=64, ssm_state_size=128, n_groups=8, conv_kernel=4, vocab_size=s["vocab"],
                layer_norm_epsilon=1e-6, max_position_embeddings=8192, time_step_min=0.001, tie_word_embeddings=True)


M_SIZES = {
    "2k": dict(width=2048, heads=16, q_rank=768, ff=5632, experts=32, top=4, eff=1024, sff=2048, vocab=32768),
    "4k": dict(width=4096, heads=32, q_rank=1536, ff=14336, experts=32, top=4, eff=2048, sff=4096, vocab=32768),
}


def metitar_config(s: dict) -> dict:
    """[latent attention + dense, hgrn2 + moe, hgrn2 + dense, latent attention on layer 0's cache + moe] x 2:
    128 + 32-wide heads over a 224-wide latent (256-wide cache rows), HGRN2 heads of 128 x 128."""
    att = {"heads": s["heads"], "dim": 128, "rot_dim": 32, "vdim": 128, "kv_rank": 224, "q_rank": s["q_rank"],
           "rot": {"base": 10000.0, "dims": 32, "scaling": {"factor": 8.0, "original": 1024, "fast": 32.0, "slow": 1.0}},
           "scale": 160 ** -0.5}
    rec = {"heads": s["heads"], "dim": 128, "vdim": 128}
    dense = {"kind": "dense", "ff": s["ff"]}
    moe = {"kind": "moe", "router": {"experts": s["experts"], "top": s["top"]}, "expert": {"ff": s["eff"]},
           "shared": {"ff": s["sff"]}}
    layers = []
    for blk in range(2):
        a0 = 4 * blk
        layers += [{"type": "latent_attention", "mixer": dict(att), "mlp": dense},
                   {"type": "hgrn2", "mixer": rec, "mlp": moe}, {"type": "hgrn2", "mixer": rec, "mlp": dense},
                   {"type": "latent_attention", "mixer": dict(att, kv_from=a0), "mlp": moe}]
    return {"architecture": "Metitar", "embedding": {"scale": 4.0}, "layers": layers, "norm": {"eps": 1e-6},
            "canon": {"taps": 4}, "token_side": {"dim": 64}, "logit_scale": 1.0, "vocab": s["vocab"],
            "width": s["width"], "max_positions": 8192}


def deepseek_like_config(s: dict) -> dict:
    """Eight MLA layers (256 + 32-wide latent cache rows: the kernel's second shape), four dense then
    four routed feed-forwards of the Metitar stack's sizes."""
    return dict(architectures=["DeepseekV2ForCausalLM"], model_type="deepseek_v2", hidden_size=s["width"],
                num_hidden_layers=8, num_attention_heads=s["heads"], num_key_value_heads=s["heads"],
                intermediate_size=s["ff"], moe_intermediate_size=s["eff"], n_routed_experts=s["experts"],
                n_shared_experts=s["sff"] // s["eff"], num_experts_per_tok=s["top"], first_k_dense_replace=4, n_group=1,
                topk_group=1, topk_method="greedy", scoring_func="softmax", norm_topk_prob=False,
                routed_scaling_factor=1.0, kv_lora_rank=256, q_lora_rank=s["q_rank"], qk_nope_head_dim=128,
                qk_rope_head_dim=32, v_head_dim=128, vocab_size=s["vocab"], rms_norm_eps=1e-6, rope_theta=10000.0,
                max_position_embeddings=8192, tie_word_embeddings=False)


X_SIZES = {
    "2k": dict(width=2048, heads=16, kv=4, experts=32, top=4, eff=1024, vocab=32768),
    "4k": dict(width=4096, heads=32, kv=8, experts=32, top=4, eff=2048, vocab=32768),
}


def milenex_config(s: dict, window: int = 1024) -> dict:
    """[talking-heads attention, conv + rotary attention] x 4, 128-wide heads, every layer with 32
    experts in 4 groups (2 kept), top 4, and a gated shared expert of an expert's width."""
    base = {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "mask": {"size": window},
            "scale": 128 ** -0.5}
    rot = dict(base, conv=4, rot={"base": 10000.0, "dims": 64})
    moe = {"kind": "moe", "router": {"experts": s["experts"], "top": s["top"], "groups": {"count": 4, "keep": 2}},
           "expert": {"ff": s["eff"], "limit": 7.0}, "shared": {"ff": s["eff"], "limit": 7.0}}
    layers = [{"type": "attention_2", "mixer": dict(base), "mlp": moe}, {"type": "attention", "mixer": rot, "mlp": moe}] * 4
    return {"architecture": "Milenex", "layers": layers, "norm": {"eps": 1e-6}, "vocab": s["vocab"],
            "width": s["width"], "max_positions": 8192}


def nivasun_config(s: dict, window: int = 1024) -> dict:
    """[differential, key-valued, differential, latent] x 2 with 128-wide heads (the differential
    layers have half the heads, each with two score maps), a 256-wide latent, 4 taps in front of every
    mixer, every layer with 32 experts, top 4, and a gated shared expert of an expert's width."""
    moe = {"kind": "moe", "router": {"experts": s["experts"], "top": s["top"]}, "expert": {"ff": s["eff"]},
           "shared": {"ff": s["eff"]}}
    mask, rot = {"size": window}, {"base": 10000.0, "dims": 64}
    dif = {"type": "attention_2", "mlp": moe,
           "mixer": {"heads": s["heads"] // 2, "kv_heads": s["kv"] // 2, "dim": 128, "vdim": 128, "mask": mask, "rot": rot,
                     "scale": 128 ** -0.5, "diff": 0.5}}
    key = {"type": "attention", "mlp": moe,
           "mixer": {"heads": s["heads"], "kv_heads": s["kv"], "dim": 128, "vdim": 128, "mask": mask, "rot": rot,
                     "scale": 128 ** -0.5}}
    lat = {"type": "latent_attention", "mlp": moe,
           "mixer": {"heads": s["heads"], "dim": 128, "vdim": 128, "kv_rank": 256, "q_rank": 768, "mask": mask,
                     "scale": 128 ** -0.5}}
    return {"architecture": "Nivasun", "layers": [dif, key, dif, lat] * 2, "norm": {"eps": 1e-6}, "vocab": s["vocab"],
            "width": s["width"], "max_positions": 8192, "canon": {"taps": 4}, "logit_softcap": 25.0,
            "embedding": {"scale": 1.0, "bigram": {"buckets": 65521, "mul_prev": 36313, "mul_cur": 27191}}}


def gpt_oss_like_config(s: dict, window: int = 1024) -> dict:
    """Eight sliding-window layers with sinks and clamped-GLU experts of the Milenex stack's sizes."""
    return dict(architectures=["GptOssForCausalLM"], model_type="gpt_oss", hidden_size=s["width"],
                num_hidden_layers=8, num_attention_heads=s["heads"], num_key_value_heads=s["kv"], head_dim=128,
                intermediate_size=s["eff"], num_local_experts=s["experts"], num_experts_per_tok=s["top"],
                vocab_size=s["vocab"], rms_norm_eps=1e-6, sliding_window=window, layer_types=["sliding_attention"] * 8,
                attention_bias=True, max_position_embeddings=8192, rope_theta=10000.0, tie_word_embeddings=False)


def _engine(name: str, cfg: dict, max_running: int, context: int):
    from ome_amd.models.config import PRESETS
    from ome_amd.runtime.engine import Engine, EngineArgs

    PRESETS[name] = cfg
    return Engine(EngineArgs(model=name, device="cuda", load_format="dummy", max_running_requests=max_running,
                             context_length=context, chunked_prefill_size=4096, max_total_tokens=max_running * context,
                             watchdog_timeout=0.0, cuda_graph_max_bs=max_running))


def throughput(name: str, cfg: dict, prefill_len: int = 2048, prefill_n: int = 8, decode_bs: int = 32,
               decode_ctx: int = 1024, decode_n: int = 64) -> dict:
    """Prefill tokens/s (``prefill_n`` prompts of ``prefill_len``, one new token each) and decode
    tokens/s (``decode_bs`` requests at ~``decode_ctx`` context, ``decode_n`` tokens each, timed
    from the last first token to the end) through the engine's scheduler and HIP-graph decode."""
    import random

    from ome_amd.runtime.request import SamplingParams

    eng = _engine(name, cfg, max(decode_bs, prefill_n), prefill_len + decode_ctx)
    g = random.Random(0)
    V = cfg.get("vocab") or cfg.get("vocab_size")

    def toks(n):
        return [g.randrange(V) for _ in range(n)]

    one = SamplingParams(max_new_tokens=1, temperature=0.0, ignore_eos=True)
    eng.generate([toks(prefill_len)], one)                       # warm-up (allocations, GEMM heuristics)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eng.generate([toks(prefill_len) for _ in range(prefill_n)], one)
    torch.cuda.synchronize()
    pre = prefill_n * prefill_len / (time.perf_counter() - t0)
    reqs = eng.generate([toks(decode_ctx) for _ in range(decode_bs)],
                        SamplingParams(max_new_tokens=decode_n + 1, temperature=0.0, ignore_eos=True))
    first = max(r.token_times[0] for r in reqs)
    last = max(r.token_times[-1] for r in reqs)
    dec = decode_bs * decode_n / max(last - first, 1e-9)
    out = {"model": name, "prefill_tok_s": round(pre), "decode_tok_s": round(dec),
           "weights_GiB": round(eng.runner.model.weight_bytes() / 2 ** 30, 2)}
    del eng
    torch.cuda.empty_cache()
    return out


def _time_us(fn, iters: int = 30) -> float:
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    s.record()
    for _ in range(iters):
        fn()
    e.record()
    e.synchronize()
    return s.elapsed_time(e) * 1000.0 / iters


def kernel_table(T: int = 4096, B: int = 64, ctx: int = 4096, width: int = 4096) -> list[dict]:
    """(kernel of the design, like kernel of an existing model) pairs at prefill (``T`` rows) and
    decode (``B`` rows, ``ctx`` context) sizes: microseconds, bytes that must move, share of the
    HBM roofline, and how much further from it the new kernel is (``vs_like`` <= 2 is the bar)."""
    from ome_amd import ops
    from ome_amd.models.config import plain_rope_table

    dev, bf = "cuda", torch.bfloat16
    rows = []

    def pair(name, new, like, bytes_new, bytes_like, note=""):
        tn, tl = _time_us(new), _time_us(like)
        fn, fl = bytes_new / tn / 1e3 / HBM_GBS, bytes_like / tl / 1e3 / HBM_GBS
        rows.append({"kernel": name, "us": round(tn, 1), "roofline": round(fn, 3), "like_us": round(tl, 1),
                     "like_roofline": round(fl, 3), "vs_like": round(fl / max(fn, 1e-9), 2), "note": note})

    torch.manual_seed(0)
    for R, tag in ((T, "prefill"), (B, "decode")):
        # ---- residual add + RMSNorm: fp32 residual vs the bf16-residual kernel
        res = torch.randn(R, width, device=dev)
        x1 = torch.randn(R, width, device=dev).to(bf)
        x2 = torch.randn(R, width, device=dev).to(bf)
        w = torch.ones(width, device=dev, dtype=bf)
        rb, xb = res.to(bf), x1.clone()
        pair(f"residual_rmsnorm 1 addend ({tag})", lambda: ops.residual_rmsnorm(res, w, 1e-6, x1, 1.0),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 12, R * width * 8,
             "fp32 residual: 12 B / element against 8")
        pair(f"residual_rmsnorm 2 addends ({tag})", lambda: ops.residual_rmsnorm(res, w, 1e-6, x1, 0.5, x2, 0.5),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 14, R * width * 8)
        # ---- q/k norm + rotary + paged write
        Hq, Hkv, D, P = 32, 8, 128, 16
        n_pages = R // P + 2
        kc = torch.zeros(n_pages, Hkv, P, D, device=dev, dtype=bf)
        vc = torch.zeros(n_pages, Hkv, D, P, device=dev, dtype=bf)
        qkv = torch.randn(R, (Hq + 2 * Hkv) * D, device=dev).to(bf)
        pos = torch.arange(R, dtype=torch.int32, device=dev)
        slots = pos + P
        cs = plain_rope_table(10000.0, 64, R + 1, dev)
        qo = torch.empty(R, Hq, D, device=dev, dtype=bf)
        qn, kn = torch.ones(Hq * D, device=dev, dtype=bf), torch.ones(Hkv * D, device=dev, dtype=bf)
        hn = torch.ones(D, device=dev, dtype=bf)
        nb = R * (Hq + 2 * Hkv) * D * 2 * 2
        pair(f"wide_norm_rope_cache ({tag})",
             lambda: ops.wide_norm_rope_cache(qkv[:, :Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D:],
                                              pos, cs, 64, True, qn, kn, 1e-6, qo, kc, vc, slots, Hq, Hkv, D, D),
             lambda: ops.rope_qkv_cache(qkv, pos, cs, 64, qo, kc, vc, slots, Hq, Hkv, D, True, hn, hn, 1e-6), nb, nb,
             "projection-wide norm: two passes over q / k")
        # ---- output gate
        o = torch.randn(R, Hq, D, device=dev).to(bf)
        gt = torch.randn(R, Hq * D, device=dev).to(bf)
        pair(f"head_gate ({tag})", lambda: ops.head_gate(o, gt, D, 0),
             lambda: o.view(R, Hq * D) * torch.sigmoid(gt), R * Hq * D * 6, R * Hq * D * 8,
             "like: the two eager elementwise kernels of the gated attention of Qwen3-Next")
        # ---- clamped GLU (same kernel, runtime limit)
        I = 14336
        gu = torch.randn(R, 2 * I, device=dev).to(bf)
        pair(f"act_and_mul limit ({tag})", lambda: ops.act_and_mul(gu, 2, limit=3.0), lambda: ops.act_and_mul(gu, 2),
             R * I * 6, R * I * 6)
    # ---- attention: decode over a long context, window + kept first keys vs the plain window
    Hq, Hkv, D, P, W = 32, 8, 128, 16, 1024
    per = ctx // P
    kc = (torch.randn(B * per + 1, Hkv, P, D, device=dev) * 0.3).to(bf)
    vc = (torch.randn(B * per + 1, Hkv, D, P, device=dev) * 0.3).to(bf)
    bt = (torch.arange(B * per, dtype=torch.int32, device=dev) + 1).view(B, per)
    sl = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q = torch.randn(B, Hq, D, device=dev).to(bf)
    ws = ops.DecodeWorkspace(B, Hq, D, ctx, 0, dev, parts=4)
    kvb = B * Hkv * D * 2 * 2
    pair("paged_decode window 1024 + 8 kept", lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W, keep_first=8),
         lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W), kvb * (W + 32), kvb * W,
         "one more 32-key tile per sequence for the kept keys")
    # ---- attention: prefill, 2 x 2048 rows
    q_lens = [2048, 2048]
    Tq = sum(q_lens)
    qp = torch.randn(Tq, Hq, D, device=dev).to(bf)
    cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
    kl = torch.tensor(q_lens, dtype=torch.int32, device=dev)
    bt2 = (torch.arange(2 * 128, dtype=torch.int32, device=dev) + 1).view(2, 128)
    items = torch.tensor(ops.prefill_work_items(q_lens, q_lens), dtype=torch.int32, device=dev)
    flops = 4.0 * Hq * D * sum(min(W + 8, i + 1) for i in range(2048)) * 2
    tn = _time_us(lambda: ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W, keep_first=8))
    tl = _time_us(lambda: ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W))
    rows.append({"kernel": "paged_prefill window 1024 + 8 kept (2 x 2048 rows)", "us": round(tn, 1),
                 "roofline": round(flops / tn / 1e6 / 2.5e3, 3), "like_us": round(tl, 1),
                 "like_roofline": round(flops / tl / 1e6 / 2.5e3, 3), "vs_like": round(tn / tl, 2),
                 "note": "share of 2.5 PFLOP/s bf16; like: the 4-wave GQA-4 kernel with a plain window"})
    return rows


def kernel_table_metitar(T: int = 4096, B: int = 64, ctx: int = 4096, width: int = 4096) -> list[dict]:
    """Metitar's kernels beside their like kernels (same columns as :func:`kernel_table`)."""
    from ome_amd import ops
    from ome_amd.models.config import yarn_rope_table
    from ome_amd.models.mixers import InputScaledMoE

    dev, bf = "cuda", torch.bfloat16
    rows = []

    def pair(name, new, like, bytes_new, bytes_like, note=""):
        tn, tl = _time_us(new), _time_us(like)
        fn, fl = bytes_new / tn / 1e3 / HBM_GBS, bytes_like / tl / 1e3 / HBM_GBS
        rows.append({"kernel": name, "us": round(tn, 1), "roofline": round(fn, 3), "like_us": round(tl, 1),
                     "like_roofline": round(fl, 3), "vs_like": round(fl / max(fn, 1e-9), 2), "note": note})

    def seqs(lens):
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        n = len(lens)
        return cu, torch.arange(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev)

    torch.manual_seed(0)
    H, d, vd = 32, 128, 128
    for R, tag, lens in ((T, "prefill", [T // 8] * 8), (B, "decode", [1] * B)):
        cu, slot, reset = seqs(lens)
        S = len(lens)
        # ---- post-norm residual add (fp32 stream, layer norm of the addend) vs add + RMSNorm on a bf16 stream
        res = torch.randn(R, width, device=dev)
        y = torch.randn(R, width, device=dev).to(bf)
        w, b = torch.ones(width, device=dev, dtype=bf), torch.zeros(width, device=dev, dtype=bf)
        rb, xb = res.to(bf), y.clone()
        pair(f"post_norm_add layer norm ({tag})", lambda: ops.post_norm_add(res, y, w, b, 1e-6, 0, bf),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 12, R * width * 8,
             "fp32 stream: 12 B / element against 8; the addend is read twice more from cache (mean, variance)")
        # ---- residual causal conv on the fp32 stream vs the conv + SiLU of the recurrent mixers
        wc = (torch.randn(width, 4, device=dev) * 0.3).to(bf)
        st32 = torch.zeros(S, width, 3, device=dev)
        stb = torch.zeros(S, width, 3, device=dev, dtype=bf)
        pair(f"conv_mix 4 taps ({tag})", lambda: ops.conv_mix(res, wc, st32, cu, slot, reset, bf),
             lambda: ops.ssm_conv1d(y, wc, None, stb, cu, slot, reset), R * width * 6, R * width * 4,
             "time-parallel tiles; like: one thread per channel walks the sequence")
        # ---- HGRN2 scan (+ activations + head norm) vs the gated delta rule scan of equal head shape
        p = torch.randn(R, 2 * H * d + H * vd, device=dev).to(bf)
        fb, lo, gw = torch.zeros(H * d, device=dev, dtype=bf), torch.full((H * d,), 0.3, device=dev, dtype=bf), \
            torch.ones(vd, device=dev, dtype=bf)
        st = torch.zeros(S, H, d, vd, device=dev)
        ab = torch.randn(R, 2 * H, device=dev).to(bf)
        Al, db = torch.zeros(H, device=dev), torch.zeros(H, device=dev)
        state_b = S * H * d * vd * 4 * 2
        io_new, io_like = R * (2 * H * d + 2 * H * vd) * 2, R * (2 * H * d + 2 * H * vd + 2 * H) * 2
        pair(f"hgrn2_scan 32 x 128 x 128 ({tag})",
             lambda: ops.hgrn2_scan(p[:, :H * d], p[:, H * d:2 * H * d], p[:, 2 * H * d:], fb, lo, gw, st, cu, slot, reset,
                                    H, d, vd, 1e-6),
             lambda: ops.gdn_scan(p[:, :H * d], p[:, H * d:2 * H * d], p[:, 2 * H * d:], ab[:, :H], ab[:, H:], Al, db, st,
                                  cu, slot, reset, H, H), state_b + io_new, state_b + io_like,
             "like: Qwen3-Next's gated delta rule (state in and out dominate decode; prefill is latency of the walk)")
        # ---- PolyNorm vs SiLU-and-mul
        I = 14336
        z = torch.randn(R, I, device=dev).to(bf)
        gu = torch.randn(R, 2 * I, device=dev).to(bf)
        coef = torch.tensor([0.9, -0.4, 0.3, 0.05], device=dev)
        pair(f"polynorm ({tag})", lambda: ops.polynorm(z, coef, 1e-6), lambda: ops.act_and_mul(gu, 0), R * I * 4,
             R * I * 6, "two passes over the row (three mean squares, then the sum)")
        # ---- latent glue vs the MLA glue
        qlr, lat, rope, D, P = 1536, 224, 32, 288, 16
        a = torch.randn(R, qlr + lat + rope, device=dev).to(bf)
        a2 = torch.randn(R, qlr + 256 + rope, device=dev).to(bf)
        nw, nw2 = torch.ones(lat, device=dev, dtype=bf), torch.ones(256, device=dev, dtype=bf)
        pos = torch.arange(R, dtype=torch.int32, device=dev) % 2048
        slots = torch.arange(R, dtype=torch.int32, device=dev) + P
        cs = yarn_rope_table(10000.0, rope, 2048, None, dev)
        q = torch.randn(R, H, 128 + rope, device=dev).to(bf)
        kc = torch.zeros(R // P + 2, 1, P, D, device=dev, dtype=bf)
        qf = torch.empty(R, H, D, device=dev, dtype=bf)
        lc = torch.zeros((R // P + 2) * P, 288, device=dev, dtype=bf)
        qf2 = torch.empty(R, H, 288, device=dev, dtype=bf)
        nb = R * ((lat + rope) * 2 * 2 + H * rope * 2 * 2)
        pair(f"latent_prep ({tag})",
             lambda: ops.latent_prep(a, qlr, lat, rope, nw, 1e-6, pos, cs, slots, kc, None, q, 128, qf, rope_off=256),
             lambda: ops.mla_prep(a2, qlr, 256, rope, nw2, 1e-6, pos, cs, slots, lc, q, 128, qf2), nb, nb,
             "same glue with a rotary offset and zero fill of the row's gaps")
        # ---- routed feed-forward, router score on the expert's input vs on its output
        E, k, ff = 32, 4, 2048
        moe = InputScaledMoE(width, E, k, ff, 0, dev, bf)
        moe.init_random(torch.Generator(device=dev).manual_seed(1), 0.02)
        x = torch.randn(R, width, device=dev).to(bf)
        lg = torch.randn(R, E, device=dev)
        tw, tid = ops.moe_route(lg, k, False, "sigmoid")
        touched = min(E, R * k) * 3 * ff * width * 2
        pair(f"input-scaled moe 32 experts top 4 ({tag})", lambda: moe.forward(x),
             lambda: ops.fused_moe(x, tw, tid, moe.w13, moe.w2, 0, 1.0), touched, touched,
             "new: router GEMM + route + row scaling + grouped GEMMs + unit-weight combine; like: grouped GEMMs + combine")
    # ---- latent attention: the 16-head MFMA latent kernel with sinks (288-wide rows: 224 latent + 32 rotary,
    # padded) vs the same kernel as DeepSeek-style MLA runs it (no sinks)
    Hq, DK, DV, P = 16, 288, 256, 16
    per = ctx // P
    lc = (torch.randn(B * per + 1, P, DK, device=dev) * 0.3).to(bf)
    bt = (torch.arange(B * per, dtype=torch.int32, device=dev) + 1).view(B, per)
    sl = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q2 = torch.randn(B, Hq, DK, device=dev).to(bf)
    sinks = torch.zeros(Hq, device=dev)
    mws = ops.MLAWorkspace(dev)
    rows_i = torch.arange(B, dtype=torch.int32, device=dev)
    pair("latent attention decode 64 x 4096 ctx, 16 heads",
         lambda: ops.latent_attn(q2, lc, bt, rows_i, sl, 0.08, DV, mws, sinks=sinks),
         lambda: ops.mla_attn(q2, lc, bt, rows_i, sl, 0.08, mws, dv=DV), B * ctx * DK * 2, B * ctx * DK * 2,
         "the latent row is read once, for keys and values")
    # ---- latent attention, prefill 2 x 2048 rows
    q_lens = [2048, 2048]
    Tq = sum(q_lens)
    qp2 = torch.randn(Tq, Hq, DK, device=dev).to(bf)
    bt2 = (torch.arange(2 * 128, dtype=torch.int32, device=dev) + 1).view(2, 128)
    tok_row = torch.arange(Tq, dtype=torch.int32, device=dev) // 2048
    tok_len = (torch.arange(Tq, dtype=torch.int32, device=dev) % 2048 + 1).to(torch.int32)
    fl = 2.0 * Hq * (DK + DV) * sum(i + 1 for i in range(2048)) * 2
    tn = _time_us(lambda: ops.latent_attn(qp2, lc, bt2, tok_row, tok_len, 0.08, DV, mws, sinks=sinks), 10)
    tl = _time_us(lambda: ops.mla_attn(qp2, lc, bt2, tok_row, tok_len, 0.08, mws, dv=DV), 10)
    rn, rl = fl / tn / 1e6 / 2.5e3, fl / tl / 1e6 / 2.5e3
    rows.append({"kernel": "latent attention prefill 2 x 2048 rows, 16 heads", "us": round(tn, 1), "roofline": round(rn, 3),
                 "like_us": round(tl, 1), "like_roofline": round(rl, 3), "vs_like": round(rl / max(rn, 1e-9), 2),
                 "note": "share of 2.5 PFLOP/s bf16; one token x 16 heads per work item"})
    return rows


def kernel_table_milenex(T: int = 4096, B: int = 64, ctx: int = 4096, width: int = 4096) -> list[dict]:
    """Milenex's kernels beside their like kernels (same columns as :func:`kernel_table`)."""
    from ome_amd import ops
    from ome_amd.models.config import plain_rope_table
    from ome_amd.models.mixers import GroupRoutedMoE

    dev, bf = "cuda", torch.bfloat16
    rows = []

    def pair(name, new, like, bytes_new, bytes_like, note="", iters=30):
        tn, tl = _time_us(new, iters), _time_us(like, iters)
        fn, fl = bytes_new / tn / 1e3 / HBM_GBS, bytes_like / tl / 1e3 / HBM_GBS
        rows.append({"kernel": name, "us": round(tn, 1), "roofline": round(fn, 3), "like_us": round(tl, 1),
                     "like_roofline": round(fl, 3), "vs_like": round(fl / max(fn, 1e-9), 2), "note": note})

    def seqs(lens):
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        n = len(lens)
        return cu, torch.arange(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev)

    torch.manual_seed(0)
    Hq, Hkv, D, P, W = 32, 8, 128, 16, 1024
    for R, tag, lens in ((T, "prefill", [T // 8] * 8), (B, "decode", [1] * B)):
        sq = seqs(lens)
        # ---- stream update + offset norm (+ token shift) vs add + RMSNorm on a bf16 stream
        res = torch.randn(R, width, device=dev)
        y = torch.randn(R, width, device=dev).to(bf)
        w, mu = torch.zeros(width, device=dev, dtype=bf), torch.rand(width, device=dev).to(bf)
        st = torch.zeros(len(lens), width, device=dev)
        rb, xb = res.to(bf), y.clone()
        pair(f"shift_norm with token shift ({tag})",
             lambda: ops.shift_norm(res, w, 1e-6, y, 1.0, None, 1.0, 1.0, mu, st, sq, bf),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 12, R * width * 8,
             "fp32 stream in and out of place: 12 B / element against 8; the row before is read again from cache")
        pair(f"shift_norm, no shift ({tag})", lambda: ops.shift_norm(res, w, 1e-6, y, w_offset=1.0, out_dtype=bf),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 12, R * width * 8)
        # ---- convolution + rotary + unit norm + paged write vs per-head norm + rotary + paged write
        n_pages = R // P + 2
        kc = torch.zeros(n_pages, Hkv, P, D, device=dev, dtype=bf)
        vc = torch.zeros(n_pages, Hkv, D, P, device=dev, dtype=bf)
        C = (Hq + 2 * Hkv) * D
        qkv = torch.randn(R, C, device=dev).to(bf)
        pos = torch.arange(R, dtype=torch.int32, device=dev) % 2048
        slots = torch.arange(R, dtype=torch.int32, device=dev) + P
        cs = plain_rope_table(10000.0, 64, 2049, dev)
        qo = torch.empty(R, Hq, D, device=dev, dtype=bf)
        cw = [(torch.randn(c, 4, device=dev) * 0.3).to(bf) for c in (Hq * D, Hkv * D, Hkv * D)]
        tail = torch.zeros(len(lens), 3, C, device=dev, dtype=bf)
        hn = torch.ones(D, device=dev, dtype=bf)
        nb = R * C * 2 * 2
        srows = ops.seq_rows(sq, R)      # (once per step in the model, shared by its layers)
        qv, kv_, vv = qkv[:, :Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D], qkv[:, (Hq + Hkv) * D:]
        pair(f"conv_rope_cache 4 taps ({tag})",
             lambda: ops.conv_rope_cache(qv, kv_, vv, *cw, tail, sq, pos, cs, 64, True, True, 1e-6, qo, kc, vc, slots,
                                         Hq, Hkv, D, D, rows=srows),
             lambda: ops.rope_qkv_cache(qkv, pos, cs, 64, qo, kc, vc, slots, Hq, Hkv, D, True, hn, hn, 1e-6), nb, nb,
             "like: Qwen3's per-head norm + rotary + cache write (no convolution)")
        # ---- clamped GLU with the shared expert's per-row gate vs without
        I = 2048
        gu = torch.randn(R, 2 * I, device=dev).to(bf)
        rg = torch.randn(R, 33, device=dev)
        pair(f"act_and_mul row gate ({tag})", lambda: ops.act_and_mul(gu, 2, limit=7.0, row_gate=rg[:, 32]),
             lambda: ops.act_and_mul(gu, 2), R * I * 6, R * I * 6)
        # ---- routed feed-forward: grouped routing + gated shared expert vs GPT-OSS's experts
        E, k, ff = 32, 4, 2048
        moe = GroupRoutedMoE(width, E, k, ff, 7.0, 4, 2, ff, 7.0, dev, bf)
        moe.init_random(torch.Generator(device=dev).manual_seed(1), 0.02)
        x = torch.randn(R, width, device=dev).to(bf)
        lg = torch.randn(R, E, device=dev)
        tw, tid = ops.moe_route(lg, k, True, "softmax")
        touched = min(E, R * k) * 3 * ff * width * 2
        pair(f"group-routed moe 32 experts top 4 + shared ({tag})", lambda: moe.forward(x),
             lambda: ops.fused_moe(x, tw, tid, moe.w13, moe.w2, 2, 1.0), touched + 3 * ff * width * 2, touched,
             "new: router GEMM + route + shared expert (3 GEMMs) + grouped GEMMs + combine; like: grouped GEMMs + combine",
             10)
    # ---- attention with mixed heads: decode over a long context vs the sliding-window decode kernel with sinks
    per = ctx // P
    kc = (torch.randn(B * per + 1, Hkv, P, D, device=dev) * 0.3).to(bf)
    vc = (torch.randn(B * per + 1, Hkv, D, P, device=dev) * 0.3).to(bf)
    bt = (torch.arange(B * per, dtype=torch.int32, device=dev) + 1).view(B, per)
    sl = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q = (torch.randn(B, Hq, D, device=dev) * 0.3).to(bf)
    gate = torch.randn(B, Hq, device=dev).to(bf)
    sinks = torch.zeros(Hq, device=dev)
    r1, r2 = torch.full((Hq,), 0.3, device=dev), torch.full((Hq,), 1.0, device=dev)
    talk = torch.eye(Hq, device=dev) + 0.05
    ws = ops.DecodeWorkspace(B, Hq, D, ctx, 0, dev, parts=4)
    rows_i = torch.arange(B, dtype=torch.int32, device=dev)
    kvb = B * Hkv * D * 2 * 2 * W
    pair("talking_attn decode 64 x 4096 ctx, window 1024",
         lambda: ops.talking_decode(q, kc, vc, bt, sl, 0.09, W, sinks, r1, r2, talk, gate, D),
         lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W, sinks=sinks), kvb, kvb,
         "three launches: pass 1 per key split, pass 2 per key split (keys read again, mix over heads), sum + gate", 10)
    pair("talking_attn row kernel (fp32 models' path, here on bf16), same shape",
         lambda: ops.talking_attn(q, kc, vc, bt, rows_i, sl - 1, 0.09, W, sinks, r1, r2, talk, gate, D),
         lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W, sinks=sinks), kvb, kvb,
         "exactness path: one workgroup per row, no matrix cores", 3)
    # ---- prefill, 2 x 2048 rows
    q_lens = [2048, 2048]
    Tq = sum(q_lens)
    qp = (torch.randn(Tq, Hq, D, device=dev) * 0.3).to(bf)
    gp = torch.randn(Tq, Hq, device=dev).to(bf)
    cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
    kl = torch.tensor(q_lens, dtype=torch.int32, device=dev)
    bt2 = (torch.arange(2 * 128, dtype=torch.int32, device=dev) + 1).view(2, 128)
    items = torch.tensor(ops.prefill_work_items(q_lens, q_lens), dtype=torch.int32, device=dev)
    flops = 4.0 * Hq * D * sum(min(W, i + 1) for i in range(2048)) * 2
    tn = _time_us(lambda: ops.talking_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W, sinks, r1, r2, talk, gp, D), 5)
    tl = _time_us(lambda: ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W, sinks=sinks), 5)
    rows.append({"kernel": "talking_attn prefill 2 x 2048 rows, window 1024", "us": round(tn, 1),
                 "roofline": round(flops / tn / 1e6 / 2.5e3, 3), "like_us": round(tl, 1),
                 "like_roofline": round(flops / tl / 1e6 / 2.5e3, 3), "vs_like": round(tn / tl, 2),
                 "note": "share of 2.5 PFLOP/s bf16 (q.k and p.v only); like: the MFMA sliding-window kernel with sinks"})
    return rows


def kernel_table_nivasun(T: int = 4096, B: int = 64, ctx: int = 4096, width: int = 4096) -> list[dict]:
    """Nivasun's kernels beside their like kernels (same columns as :func:`kernel_table`)."""
    from ome_amd import ops
    from ome_amd.models.config import plain_rope_table
    from ome_amd.models.mixers import GroupRoutedMoE

    dev, bf = "cuda", torch.bfloat16
    rows = []

    def pair(name, new, like, bytes_new, bytes_like, note="", iters=30):
        tn, tl = _time_us(new, iters), _time_us(like, iters)
        fn, fl = bytes_new / tn / 1e3 / HBM_GBS, bytes_like / tl / 1e3 / HBM_GBS
        rows.append({"kernel": name, "us": round(tn, 1), "roofline": round(fn, 3), "like_us": round(tl, 1),
                     "like_roofline": round(fl, 3), "vs_like": round(fl / max(fn, 1e-9), 2), "note": note})

    def seqs(lens):
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        n = len(lens)
        return cu, torch.arange(n, dtype=torch.int32, device=dev), torch.zeros(n, dtype=torch.int32, device=dev)

    torch.manual_seed(0)
    Hq, Hkv, D, P, W = 32, 8, 128, 16, 1024
    for R, tag, lens in ((T, "prefill", [T // 8] * 8), (B, "decode", [1] * B)):
        sq = seqs(lens)
        # ---- token-pair embedding vs the plain embedding
        V = 32768
        ids = torch.randint(0, V, (R,), dtype=torch.int32, device=dev)
        emb, prs = torch.randn(V, width, device=dev).to(bf), torch.randn(65522, width, device=dev).to(bf)
        prev = torch.zeros(len(lens) + 1, dtype=torch.int32, device=dev)
        pair(f"pair_embedding_f32 ({tag})",
             lambda: ops.pair_embedding_f32(ids, emb, 1.0, prs, 65521, 36313, 27191, prev, sq),
             lambda: ops.embedding(ids, emb), R * width * 8, R * width * 4,
             "two table rows in, an fp32 row out: 8 B / element against 4")
        # ---- stream update with two addends and a pass vector + single-gain norm vs add + RMSNorm on a bf16 stream
        res = torch.randn(R, width, device=dev)
        y1, y2 = torch.randn(R, width, device=dev).to(bf), torch.randn(R, width, device=dev).to(bf)
        w, step = torch.ones(width, device=dev, dtype=bf), torch.randn(width, device=dev).to(bf)
        rb, xb = res.to(bf), y1.clone()
        pair(f"shift_norm, two addends + pass vector ({tag})",
             lambda: ops.shift_norm(res, w, 1e-6, y1, 1.0, y2, 1.0, out_dtype=bf, bias=step),
             lambda: ops.fused_add_rmsnorm(xb, rb, w, 1e-6), R * width * 14, R * width * 8,
             "fp32 stream + two sublayer outputs: 14 B / element against 8")
        # ---- residual convolution of the normed rows vs the causal conv of the recurrent mixers
        h = torch.randn(R, width, device=dev).to(bf)
        cw = (torch.randn(width, 4, device=dev) * 0.3).to(bf)
        st32 = torch.zeros(len(lens), width, 3, device=dev)
        stb = torch.zeros(len(lens), width, 3, device=dev, dtype=bf)
        pair(f"conv_mix 4 taps on normed rows ({tag})", lambda: ops.conv_mix(h, cw, st32, *sq, bf),
             lambda: ops.ssm_conv1d(h, cw, None, stb, *sq), R * width * 4, R * width * 4,
             "like: the depthwise conv + SiLU of Mamba-2 / delta-rule inputs")
        # ---- rotary + temperature + keys stored as values / values shared by two key heads vs Qwen3's prep
        n_pages = R // P + 2
        kc = torch.zeros(n_pages, Hkv, P, D, device=dev, dtype=bf)
        vc = torch.zeros(n_pages, Hkv, D, P, device=dev, dtype=bf)
        C = (Hq + 2 * Hkv) * D
        qkv = torch.randn(R, C, device=dev).to(bf)
        pos = torch.arange(R, dtype=torch.int32, device=dev) % 2048
        slots = torch.arange(R, dtype=torch.int32, device=dev) + P
        cs = plain_rope_table(10000.0, 64, 2049, dev)
        qo = torch.empty(R, Hq, D, device=dev, dtype=bf)
        hn = torch.ones(D, device=dev, dtype=bf)
        temp = torch.rand(Hq, device=dev) + 0.5
        qv, kv_ = qkv[:, :Hq * D], qkv[:, Hq * D:(Hq + Hkv) * D]
        like = lambda: ops.rope_qkv_cache(qkv, pos, cs, 64, qo, kc, vc, slots, Hq, Hkv, D, True, hn, hn, 1e-6)   # noqa: E731
        pair(f"wide_norm_rope_cache, half-split pairs + temperature, v = k ({tag})",
             lambda: ops.wide_norm_rope_cache(qv, kv_, kv_, pos, cs, 64, False, None, None, 0.0, qo, kc, vc, slots, Hq,
                                              Hkv, D, D, q_scale=temp),
             like, R * ((Hq + Hkv) * D * 2 + (Hq + 2 * Hkv) * D * 2), R * C * 2 * 2,
             "like: Qwen3's per-head norm + rotary + cache write")
        vh = qkv[:, (Hq + Hkv) * D:(Hq + Hkv) * D + (Hkv // 2) * D]
        pair(f"wide_norm_rope_cache, interleaved pairs, values under two key heads ({tag})",
             lambda: ops.wide_norm_rope_cache(qv, kv_, vh, pos, cs, 64, True, None, None, 0.0, qo, kc, vc, slots, Hq,
                                              Hkv, D, D, v_rep=2),
             like, R * ((Hq + Hkv + Hkv // 2) * D * 2 + (Hq + 2 * Hkv) * D * 2), R * C * 2 * 2)
        # ---- combine of the two maps + head norm vs the sigmoid head gate
        a = torch.randn(R, Hq, D, device=dev).to(bf)
        gate = torch.randn(R, Hq * D, device=dev).to(bf)
        pair(f"diff_head_norm ({tag})", lambda: ops.diff_head_norm(a, 0.6, 1e-6, 0.5, 4, D),
             lambda: ops.head_gate(a, gate, D, 0), R * Hq * D * 3, R * Hq * D * 6,
             "reads 2 heads, writes 1; like: Zavilorn's output gate (reads 2, writes 1 per head)")
        # ---- routed feed-forward: biased router + softmax over the chosen + gated shared expert vs GPT-OSS's experts
        E, k, ff = 32, 4, 2048
        moe = GroupRoutedMoE(width, E, k, ff, 0.0, 1, 1, ff, 0.0, dev, bf, act=0, renorm=True, router_bias=True,
                             correction=False)
        moe.init_random(torch.Generator(device=dev).manual_seed(1), 0.02)
        x = torch.randn(R, width, device=dev).to(bf)
        lg = torch.randn(R, E, device=dev)
        tw, tid = ops.moe_route(lg, k, True, "softmax")
        touched = min(E, R * k) * 3 * ff * width * 2
        pair(f"biased-router moe 32 experts top 4 + shared ({tag})", lambda: moe.forward(x),
             lambda: ops.fused_moe(x, tw, tid, moe.w13, moe.w2, 2, 1.0), touched + 3 * ff * width * 2, touched,
             "new: router GEMM + route + shared expert (3 GEMMs) + grouped GEMMs + combine; like: grouped GEMMs + combine",
             10)
    # ---- decode over a long context, window 1024
    per = ctx // P
    kc = (torch.randn(B * per + 1, Hkv, P, D, device=dev) * 0.3).to(bf)
    vc = (torch.randn(B * per + 1, Hkv, D, P, device=dev) * 0.3).to(bf)
    bt = (torch.arange(B * per, dtype=torch.int32, device=dev) + 1).view(B, per)
    sl = torch.full((B,), ctx, dtype=torch.int32, device=dev)
    q = (torch.randn(B, Hq, D, device=dev) * 0.3).to(bf)
    sinks = torch.zeros(Hq, device=dev)
    ws = ops.DecodeWorkspace(B, Hq, D, ctx, 0, dev, parts=4)
    kvb = B * Hkv * D * 2 * 2 * W
    like_dec = lambda: ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W, sinks=sinks)   # noqa: E731
    pair("differential attention decode 64 x 4096 ctx: 16 heads x 2 maps over 4 x 2 key heads + combine",
         lambda: ops.diff_head_norm(ops.paged_decode(q, kc, vc, bt, sl, 0.09, ws, W), 0.6, 1e-6, 0.5, 4, D), like_dec,
         B * (Hkv * D * 2 + (Hkv // 2) * D * 2) * W, kvb,
         "the values of a kv group sit under both of its key heads: 4/3 of the bytes that must move", 10)
    pair("key-valued attention decode (sinks, temperature folded into q): the like kernel's own launch",
         like_dec, like_dec, kvb, kvb, "", 10)
    R_, H_ = 256, 32
    DK, DV = ops.latent_shape(R_, 0)
    lc = (torch.randn(B * per + 1, P, DK, device=dev) * 0.3).to(bf)
    ql = (torch.randn(B, H_, DK, device=dev) * 0.3).to(bf)
    rows_i = torch.arange(B, dtype=torch.int32, device=dev)
    slw = torch.full((B,), W, dtype=torch.int32, device=dev)
    mws = ops.MLAWorkspace(dev)
    pair("latent attention decode, window 1024 of 4096 ctx (288-wide rows)",
         lambda: ops.latent_attn(ql, lc, bt, rows_i, sl, 0.09, DV, mws, window=W),
         lambda: ops.latent_attn(ql, lc, bt, rows_i, slw, 0.09, DV, mws), B * W * DK * 2, B * W * DK * 2,
         "like: the same kernel without a window over a 1024-token context", 10)
    # ---- prefill, 2 x 2048 rows
    q_lens = [2048, 2048]
    Tq = sum(q_lens)
    qp = (torch.randn(Tq, Hq, D, device=dev) * 0.3).to(bf)
    cu = torch.tensor([0, 2048, 4096], dtype=torch.int32, device=dev)
    kl = torch.tensor(q_lens, dtype=torch.int32, device=dev)
    bt2 = (torch.arange(2 * 128, dtype=torch.int32, device=dev) + 1).view(2, 128)
    items = torch.tensor(ops.prefill_work_items(q_lens, q_lens), dtype=torch.int32, device=dev)
    flops = 4.0 * Hq * D * sum(min(W, i + 1) for i in range(2048)) * 2
    tn = _time_us(lambda: ops.diff_head_norm(ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W), 0.6, 1e-6, 0.5,
                                             4, D), 5)
    tl = _time_us(lambda: ops.paged_prefill(qp, kc, vc, bt2, cu, kl, items, 0.09, W, sinks=sinks), 5)
    rows.append({"kernel": "differential attention prefill 2 x 2048 rows, window 1024 (+ combine)", "us": round(tn, 1),
                 "roofline": round(flops / tn / 1e6 / 2.5e3, 3), "like_us": round(tl, 1),
                 "like_roofline": round(flops / tl / 1e6 / 2.5e3, 3), "vs_like": round(tn / tl, 2),
                 "note": "share of 2.5 PFLOP/s bf16 (q.k and p.v only); like: the MFMA sliding-window kernel with sinks"})
    qlp = (torch.randn(Tq, H_, DK, device=dev) * 0.3).to(bf)
    tok_row = torch.arange(Tq, dtype=torch.int32, device=dev) // 2048
    lens_p = (torch.arange(Tq, dtype=torch.int32, device=dev) % 2048) + 1
    lflops = 2.0 * H_ * (DK + DV) * 2
    tn = _time_us(lambda: ops.latent_attn(qlp, lc, bt2, tok_row, lens_p, 0.09, DV, mws, window=W), 5)
    tl = _time_us(lambda: ops.latent_attn(qlp, lc, bt2, tok_row, lens_p, 0.09, DV, mws), 5)
    fw, fa = lflops * sum(min(W, i + 1) for i in range(2048)), lflops * sum(i + 1 for i in range(2048))
    rows.append({"kernel": "latent attention prefill 2 x 2048 rows, window 1024", "us": round(tn, 1),
                 "roofline": round(fw / tn / 1e6 / 2.5e3, 3), "like_us": round(tl, 1),
                 "like_roofline": round(fa / tl / 1e6 / 2.5e3, 3), "vs_like": round((fa / tl) / (fw / tn), 2),
                 "note": "like: the same kernel without a window (all 2048 keys); both as share of 2.5 PFLOP/s"})
    return rows


def run(sizes=("2k", "4k"), kernels: bool = True, only: str | None = None, design: str = "zavilorn") -> dict:
    out = {"throughput": [], "kernels": []}
    if design == "nivasun":
        for k in sizes:
            s = X_SIZES[k]
            if only in (None, "nivasun"):
                out["throughput"].append(throughput(f"nivasun-{k}", nivasun_config(s)))
            if only in (None, "gpt-oss"):
                out["throughput"].append(throughput(f"gpt-oss-like-{k}", gpt_oss_like_config(s)))
        if kernels:
            out["kernels"] = kernel_table_nivasun()
        return out
    if design == "milenex":
        for k in sizes:
            s = X_SIZES[k]
            if only in (None, "milenex"):
                out["throughput"].append(throughput(f"milenex-{k}", milenex_config(s)))
            if only in (None, "gpt-oss"):
                out["throughput"].append(throughput(f"gpt-oss-like-{k}", gpt_oss_like_config(s)))
        if kernels:
            out["kernels"] = kernel_table_milenex()
        return out
    if design == "metitar":
        for k in sizes:
            s = M_SIZES[k]
            if only in (None, "metitar"):
                out["throughput"].append(throughput(f"metitar-{k}", metitar_config(s)))
            if only in (None, "deepseek"):
                out["throughput"].append(throughput(f"deepseek-like-{k}", deepseek_like_config(s)))
        if kernels:
            out["kernels"] = kernel_table_metitar()
        return out
    for k in sizes:
        s = SIZES[k]
        if only in (None, "zavilorn"):
            out["throughput"].append(throughput(f"zavilorn-{k}", zavilorn_config(s)))
        if only in (None, "nemotron"):
            out["throughput"].append(throughput(f"nemotron-h-like-{k}", nemotron_config(s)))
    if kernels:
        out["kernels"] = kernel_table()
    return out


def main(argv=None) -> int:
    import argparse

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--sizes", default="2k,4k")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--only", choices=["zavilorn", "nemotron", "metitar", "deepseek", "milenex", "gpt-oss", "nivasun"],
                    default=None,
                    help="one stack (for kernel traces)")
    ap.add_argument("--design", choices=["zavilorn", "metitar", "milenex", "nivasun"], default="zavilorn")
    ap.add_argument("--no-throughput", action="store_true", help="the kernel table only")
    a = ap.parse_args(argv)
    res = run(() if a.no_throughput else tuple(a.sizes.split(",")), not a.no_kernels, a.only, a.design)
    for r in res["throughput"]:
        print(json.dumps(r))
    for r in res["kernels"]:
        print(json.dumps(r))
    return 0


if __name__ == "__main__":   # (run as a file under a profiler: make the package importable)
    import os
    import sys

    sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__)))))
    sys.exit(main())
