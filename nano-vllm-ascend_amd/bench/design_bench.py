"""Prefill and decode throughput of a model design beside the framework's closest existing model at equal size
(`python bench.py --design gazutar | zedirax | felolorn | sanevik`): random weights, layer sizes that resemble a real model's, both models through the same
engine entry points (add_request / step), each served the way the framework serves it (Qwen3-MoE: captured prefill and
decode steps; Gazutar: what ModelRunner reports in `served_as`).

One JSON line: per size, per model: prefill tokens/s (all prompts, wall clock around the prefill steps), decode tokens/s and
ms per decode step (wall clock around `steps` engine steps of the full batch), weight bytes a decode step streams and the
fraction of the 8 TB/s HBM roofline that makes.
"""
from __future__ import annotations

import json
import random
import time

HBM_BYTES_PER_S = 8.0e12

# (name, width, layers, heads, kv heads, head dim, experts, expert ff, top k, vocab, window)
SIZES = {
    "w1024": dict(width=1024, layers=4, heads=8, kv_heads=4, dim=128, experts=32, ff=512, top=4, vocab=32768, window=512),
    "w2048": dict(width=2048, layers=4, heads=16, kv_heads=8, dim=128, experts=64, ff=768, top=8, vocab=32768, window=1024),
}


def gazutar_config(s: dict) -> dict:
    att = {"type": "attention", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"], "vdim": s["dim"],
                                          "mask": {"size": s["window"]}, "scale": s["dim"] ** -0.5, "v_mix": True}}
    rec = {"type": "channel_delta", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": s["dim"],
                                              "vdim": s["dim"], "conv": 4, "rank": s["width"] // 16}}
    ff = {"kind": "moe", "expert": {"ff": s["ff"]},
          "router": {"experts": s["experts"], "identity": 0, "top": s["top"], "groups": {"count": 4, "keep": 2}}}
    layers = [dict(rec if i % 2 == 0 else att, mlp=ff) for i in range(s["layers"])]
    return {"architecture": "Gazutar", "vocab": s["vocab"], "width": s["width"], "logit_scale": 1.0, "norm": {"eps": 1e-6},
            "layers": layers}


def zedirax_config(s: dict) -> dict:
    """Recurrence / biased attention / recurrence / latent attention, sparse feed-forwards with a shared expert of one
    expert's size (the third layer: a dense gated one of two model widths).  The latent attention caches 192 + 64 channels
    per token for all heads."""
    W, D = s["width"], s["dim"]
    rec = {"type": "mingru", "mixer": {"width": W}}
    att = {"type": "attention", "mixer": {"heads": s["heads"], "kv_heads": s["kv_heads"], "dim": D, "vdim": D, "scale": D ** -0.5,
                                          "q_temp": {"coef": 0.1, "every": 512}}}
    lat = {"type": "latent_attention", "mixer": {"heads": s["heads"], "dim": D, "rot_dim": 64, "vdim": D, "kv_rank": 192,
                                                 "scale": (D + 64) ** -0.5, "rot": {"base": 10000.0, "dims": 64}}}
    moe = {"kind": "moe", "expert": {"ff": s["ff"]}, "router": {"experts": s["experts"], "top": s["top"]}, "shared": {"ff": s["ff"]}}
    dense = {"kind": "dense", "ff": 2 * W}
    order = [(rec, moe), (att, moe), (rec, dense), (lat, moe)]
    layers = [dict(order[i % 4][0], mlp=order[i % 4][1]) for i in range(s["layers"])]
    return {"architecture": "Zedirax", "vocab": s["vocab"], "width": W, "residual_mult": 0.5, "norm": {"eps": 1e-6}, "layers": layers}


def zedirax_decode_weight_bytes(cfg: dict, batch: int) -> float:
    """bf16 weight bytes one decode step of `batch` rows streams (every projection, the experts the rows can reach, head)."""
    W, n = cfg["width"], 0
    for l in cfg["layers"]:
        m = l["mixer"]
        if l["type"] == "mingru":
            n += 4 * W * m["width"]
        elif l["type"] == "attention":
            n += W * (m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"])) + m["heads"] * m["vdim"] * W
        else:
            H, D, R, Dv, C = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            n += W * (H * (D + R) + C + R + H * Dv) + H * C * (D + Dv) + H * Dv * W
        ml = l["mlp"]
        if ml["kind"] == "dense":
            n += 3 * W * ml["ff"]
        else:
            hit = min(ml["router"]["experts"], batch * ml["router"]["top"])
            n += hit * 2 * W * ml["expert"]["ff"] + (ml["router"]["experts"] + 1) * W + 2 * W * ml["shared"]["ff"]
    return 2.0 * (n + cfg["vocab"] * W)


def felolorn_config(s: dict) -> dict:
    """Forget-gate linear attention / latent attention / head-decay linear attention / latent attention, every layer with
    a group-routed sparse feed-forward (four groups, two kept).  The latent attention caches 256 channels per token for
    all heads (what the Zedirax bench model caches), queries through a latent of half the model width."""
    W, D, H = s["width"], s["dim"], s["heads"]
    lat = {"type": "latent_attention", "mixer": {"heads": H, "dim": D, "vdim": D, "kv_rank": 256, "q_rank": W // 2, "scale": D ** -0.5}}
    lin = {"type": "lightning", "mixer": {"heads": H, "dim": D, "vdim": D, "decay": [1.0 - 2.0 ** (-5 - 3 * h / H) for h in range(H)]}}
    fgt = {"type": "hgrn2", "mixer": {"heads": H, "dim": D, "vdim": D}}
    moe = {"kind": "moe", "expert": {"ff": s["ff"]},
           "router": {"experts": s["experts"], "top": s["top"], "groups": {"count": 4, "keep": 2}}}
    order = [fgt, lat, lin, lat]
    return {"architecture": "Felolorn", "vocab": s["vocab"], "width": W, "norm": {"eps": 1e-6}, "canon": {"taps": 4},
            "embedding": {"scale": W ** 0.5}, "logit_softcap": 30.0,
            "layers": [dict(order[i % 4], mlp=moe) for i in range(s["layers"])]}


def felolorn_decode_weight_bytes(cfg: dict, batch: int) -> float:
    """bf16 weight bytes one decode step of `batch` rows streams (every projection incl. the two residual gates, the experts
    the rows can reach, the tied table as the head)."""
    W, n = cfg["width"], 0
    for l in cfg["layers"]:
        m = l["mixer"]
        H, D, Dv = m["heads"], m["dim"], m["vdim"]
        n += W * W                                                   # the mixer's residual gate
        if l["type"] == "latent_attention":
            C, Q = m["kv_rank"], m["q_rank"]
            n += W * (Q + C) + Q * H * D + H * C * (D + Dv) + H * Dv * W
        elif l["type"] == "lightning":
            n += W * (2 * H * D + 2 * H * Dv) + H * Dv * W
        else:
            n += W * (2 * H * D + H * Dv) + H * Dv * W
        ml = l["mlp"]
        if ml is not None:
            hit = min(ml["router"]["experts"], batch * ml["router"]["top"])
            n += W * W + hit * 3 * W * ml["expert"]["ff"] + ml["router"]["experts"] * W
    return 2.0 * (n + cfg["vocab"] * W)


def sanevik_config(s: dict) -> dict:
    """Sink attention / parallel (capped, head-mixed window attention beside a retention, half of the heads each) /
    sink attention / parallel, the last two layers run twice (six layer runs per step, each with pages and state of its
    own); every layer with a sparse feed-forward whose experts take their weight on the input."""
    W, D, H, G = s["width"], s["dim"], s["heads"], s["kv_heads"]
    att = {"type": "attention",
           "mixer": {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask": {"size": s["window"]}, "scale": 1.25 * D ** -0.5,
                     "rot": {"base": 10000.0, "dims": D // 2,
                             "scaling": {"factor": 4.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}}
    par = {"type": "parallel",
           "mixer": {"left": {"heads": H // 2, "kv_heads": G // 2, "dim": D, "vdim": D, "mask": {"size": s["window"]},
                              "scale": D ** -0.5, "softcap": 30.0, "conv": 4, "rot": {"base": 10000.0, "dims": D}},
                     "right": {"heads": H // 2, "dim": D, "vdim": D, "rot": {"base": 100000.0, "dims": D // 2},
                               "decay": [1.0 - 2.0 ** (-5 - 6 * h / H) for h in range(H // 2)]},
                     "left_scale": 1.0, "right_scale": 0.5}}
    moe = {"kind": "moe", "expert": {"ff": s["ff"], "limit": 7.0}, "router": {"experts": s["experts"], "top": s["top"]}}
    order = [att, par]
    n = s["layers"]
    return {"architecture": "Sanevik", "vocab": s["vocab"], "width": W, "norm": {"eps": 1e-6},
            "loop": {"start": n - 2, "stop": n, "times": 2}, "layers": [dict(order[i % 2], mlp=moe) for i in range(n)]}


def sanevik_decode_weight_bytes(cfg: dict, batch: int) -> float:
    """bf16 weight bytes one decode step of `batch` rows streams: every projection and the experts the rows can reach, once
    per RUN of a layer (a looped layer's weights are read again in every pass), the tied table as the head."""
    W, n = cfg["width"], 0
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    for i, l in enumerate(cfg["layers"]):
        m = l["mixer"]
        if l["type"] == "attention":
            mix = W * (m["heads"] * m["dim"] + m["kv_heads"] * (m["dim"] + m["vdim"])) + m["heads"] * m["vdim"] * W
        else:
            a, r = m["left"], m["right"]
            mix = W * (a["heads"] * a["dim"] + a["kv_heads"] * (a["dim"] + a["vdim"]) + 2 * r["heads"] * (r["dim"] + r["vdim"]))
            mix += (a["heads"] * a["vdim"] + r["heads"] * r["vdim"]) * W
        ml = l["mlp"]
        if ml is not None:
            hit = min(ml["router"]["experts"], batch * ml["router"]["top"])
            mix += hit * 3 * W * ml["expert"]["ff"] + ml["router"]["experts"] * W
        n += mix * (loop["times"] if loop["start"] <= i < loop["stop"] else 1)
    return 2.0 * (n + cfg["vocab"] * W)


def qwen3_moe_config(s: dict) -> dict:
    return dict(architectures=["Qwen3MoeForCausalLM"], model_type="qwen3_moe", hidden_size=s["width"],
                num_hidden_layers=s["layers"], num_attention_heads=s["heads"], num_key_value_heads=s["kv_heads"],
                head_dim=s["dim"], intermediate_size=4 * s["width"], vocab_size=s["vocab"], max_position_embeddings=8192,
                rms_norm_eps=1e-6, rope_theta=1000000.0, tie_word_embeddings=False, attention_bias=False, hidden_act="silu",
                torch_dtype="bfloat16", bos_token_id=0, eos_token_id=s["vocab"] - 1, num_experts=s["experts"],
                num_experts_per_tok=s["top"], moe_intermediate_size=s["ff"], decoder_sparse_step=1, mlp_only_layers=[],
                norm_topk_prob=True)


def decode_weight_bytes(s: dict, batch: int, gazutar: bool) -> float:
    """bf16 weight bytes one decode step of `batch` rows streams: projections, the experts the rows can reach, head."""
    W, D, H, G = s["width"], s["dim"], s["heads"], s["kv_heads"]
    experts_hit = min(s["experts"], batch * s["top"])
    ff = experts_hit * 3 * W * s["ff"] + s["experts"] * W
    if gazutar:
        att = W * (2 * H * D + 2 * G * D) + H * D * W                 # q, g, k, v, o
        r = W // 16
        rec = W * (2 * G * D + H * D) + W * (2 * r + H) + r * 2 * H * D + H * D * W
        mix = (s["layers"] // 2) * (att + rec)
    else:
        mix = s["layers"] * (W * (H * D + 2 * G * D) + H * D * W)
    return 2.0 * (mix + s["layers"] * ff + s["vocab"] * W)


def run_model(cfg: dict, batch: int, prompt_len: int, steps: int, warmup: int, **engine_kw) -> dict:
    import torch

    from nanovllm import LLM, SamplingParams

    block = 64
    blocks = batch * ((prompt_len + steps + warmup + 8) // block + 2) + 8
    llm = LLM.from_config_dict(cfg, kvcache_block_size=block, max_num_seqs=batch, max_model_len=2 * prompt_len + 256,
                               max_num_batched_tokens=8192, num_kvcache_blocks=blocks, synthetic_seed=0, sampling_seed=0,
                               warmup=False, **engine_kw)
    try:
        vocab = llm._vocab()
        rng = random.Random(0)
        def prefill_all(max_tokens: int):
            sp = SamplingParams(temperature=1.0, max_tokens=max_tokens, ignore_eos=True, greedy=True)
            seqs = [llm.add_request([rng.randrange(vocab) for _ in range(prompt_len)], sp) for _ in range(batch)]
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            while any(s.num_completion_tokens == 0 for s in seqs):
                llm.step()
            torch.cuda.synchronize()
            return seqs, time.perf_counter() - t0

        for _ in range(2):                           # two untimed passes: allocator growth, steps captured on second sight
            prefill_all(2)
            while not llm.is_finished():
                llm.step()
        seqs, t_prefill = prefill_all(steps + warmup + 4)
        for _ in range(warmup):
            llm.step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            llm.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        runner = llm.model_runner
        served = ("eager launches (row steps)" if getattr(runner, "hybrid", False) and not getattr(runner, "row_graphs", None)
                  else "captured steps (hipGraph)")
        return {"prefill_tok_s": batch * prompt_len / t_prefill, "prefill_ms": t_prefill * 1e3,
                "decode_tok_s": batch * steps / dt, "ms_per_decode_step": dt / steps * 1e3, "served_as": served}
    finally:
        llm.exit()


def main(args) -> dict:
    batch, prompt_len = 32, 1024
    design = getattr(args, "design", None) or "gazutar"
    if design == "zedirax":
        return main_zedirax(args, batch, prompt_len)
    if design == "felolorn":
        return main_felolorn(args, batch, prompt_len)
    if design == "sanevik":
        return main_sanevik(args, batch, prompt_len)
    out = {"metric": "design_throughput", "design": "gazutar", "closest_model": "Qwen3MoeForCausalLM", "unit": "tokens/s",
           "dtype": "bf16", "data": "synthetic (random weights, random prompts)", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "batch": batch, "prompt_len": prompt_len, "sizes": {}}
    only_sizes = [x for x in getattr(args, "design_sizes", "").split(",") if x]
    only_models = [x for x in getattr(args, "design_models", "").split(",") if x]
    for name, s in SIZES.items():
        if only_sizes and name not in only_sizes:
            continue
        entry = {"shape": s}
        for label, cfg, is_g in (("gazutar", gazutar_config(s), True), ("qwen3_moe", qwen3_moe_config(s), False)):
            if only_models and label not in only_models:
                continue
            r = run_model(cfg, batch, prompt_len, args.steps, args.warmup)
            wb = decode_weight_bytes(s, batch, is_g)
            r["decode_weight_bytes"] = wb
            r["decode_weight_roofline_frac"] = wb / (r["ms_per_decode_step"] * 1e-3) / HBM_BYTES_PER_S
            entry[label] = r
        if "gazutar" in entry and "qwen3_moe" in entry:
            entry["gazutar_vs_qwen3_moe"] = {k: entry["gazutar"][k] / entry["qwen3_moe"][k] for k in ("prefill_tok_s", "decode_tok_s")}
        out["sizes"][name] = entry
    print(json.dumps(out), flush=True)
    return out


def main_zedirax(args, batch: int, prompt_len: int) -> dict:
    """Zedirax beside Gazutar - the closest existing model: the same row-step engine path, fp32 residual, pages plus state
    slots, alternating recurrent and attention mixers, sparse feed-forwards - at equal width, depth, heads, experts and
    vocabulary; Qwen3-MoE at that size rides along (`--design-models` picks)."""
    out = {"metric": "design_throughput", "design": "zedirax", "closest_model": "Gazutar", "unit": "tokens/s",
           "dtype": "bf16", "data": "synthetic (random weights, random prompts)", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "batch": batch, "prompt_len": prompt_len, "sizes": {}}
    only_sizes = [x for x in getattr(args, "design_sizes", "").split(",") if x]
    only_models = [x for x in getattr(args, "design_models", "").split(",") if x] or ["zedirax", "gazutar"]
    for name, s in SIZES.items():
        if only_sizes and name not in only_sizes:
            continue
        entry = {"shape": s}
        zc = zedirax_config(s)
        for label, cfg, wb in (("zedirax", zc, zedirax_decode_weight_bytes(zc, batch)),
                               ("gazutar", gazutar_config(s), decode_weight_bytes(s, batch, True)),
                               ("qwen3_moe", qwen3_moe_config(s), decode_weight_bytes(s, batch, False))):
            if label not in only_models:
                continue
            r = run_model(cfg, batch, prompt_len, args.steps, args.warmup)
            r["decode_weight_bytes"] = wb
            r["decode_weight_roofline_frac"] = wb / (r["ms_per_decode_step"] * 1e-3) / HBM_BYTES_PER_S
            entry[label] = r
        if "zedirax" in entry and "gazutar" in entry:
            entry["zedirax_vs_gazutar"] = {k: entry["zedirax"][k] / entry["gazutar"][k] for k in ("prefill_tok_s", "decode_tok_s")}
        out["sizes"][name] = entry
    print(json.dumps(out), flush=True)
    return out


def main_felolorn(args, batch: int, prompt_len: int) -> dict:
    """Felolorn beside Zedirax - the closest existing model: the same row-step engine path, fp32 residual with RMS norms,
    a latent attention with one cached row per token, a recurrence in state slots, sparse feed-forwards - at equal width,
    depth, heads, experts and vocabulary; Gazutar (the matrix-state recurrence and the group-limited router of the
    framework) and Qwen3-MoE at that size ride along (`--design-models` picks)."""
    out = {"metric": "design_throughput", "design": "felolorn", "closest_model": "Zedirax", "unit": "tokens/s",
           "dtype": "bf16", "data": "synthetic (random weights, random prompts)", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "batch": batch, "prompt_len": prompt_len, "sizes": {}}
    only_sizes = [x for x in getattr(args, "design_sizes", "").split(",") if x]
    only_models = [x for x in getattr(args, "design_models", "").split(",") if x] or ["felolorn", "zedirax", "gazutar"]
    for name, s in SIZES.items():
        if only_sizes and name not in only_sizes:
            continue
        entry = {"shape": s}
        fc, zc = felolorn_config(s), zedirax_config(s)
        for label, cfg, wb in (("felolorn", fc, felolorn_decode_weight_bytes(fc, batch)),
                               ("zedirax", zc, zedirax_decode_weight_bytes(zc, batch)),
                               ("gazutar", gazutar_config(s), decode_weight_bytes(s, batch, True)),
                               ("qwen3_moe", qwen3_moe_config(s), decode_weight_bytes(s, batch, False))):
            if label not in only_models:
                continue
            r = run_model(cfg, batch, prompt_len, args.steps, args.warmup)
            r["decode_weight_bytes"] = wb
            r["decode_weight_roofline_frac"] = wb / (r["ms_per_decode_step"] * 1e-3) / HBM_BYTES_PER_S
            entry[label] = r
        for other in ("zedirax", "gazutar"):
            if "felolorn" in entry and other in entry:
                entry["felolorn_vs_" + other] = {k: entry["felolorn"][k] / entry[other][k] for k in ("prefill_tok_s", "decode_tok_s")}
        out["sizes"][name] = entry
    print(json.dumps(out), flush=True)
    return out


def main_sanevik(args, batch: int, prompt_len: int) -> dict:
    """Sanevik beside Gazutar - the closest existing model: the same row-step engine path, fp32 residual, sliding-window
    attention over paged K / V rows alternating with a matrix-state recurrence behind short convolutions, sparse
    feed-forwards - at equal width, depth, heads, experts and vocabulary; Felolorn (sink softmax, head-decay linear
    attention) and Qwen3-MoE at that size ride along (`--design-models` picks).  Sanevik runs its last two layers twice:
    six layer runs per step against the others' four (`layer_runs` in the record)."""
    out = {"metric": "design_throughput", "design": "sanevik", "closest_model": "Gazutar", "unit": "tokens/s",
           "dtype": "bf16", "data": "synthetic (random weights, random prompts)", "n_gpus": 1, "steps": args.steps,
           "warmup": args.warmup, "batch": batch, "prompt_len": prompt_len, "sizes": {}}
    only_sizes = [x for x in getattr(args, "design_sizes", "").split(",") if x]
    only_models = [x for x in getattr(args, "design_models", "").split(",") if x] or ["sanevik", "gazutar", "felolorn"]
    for name, s in SIZES.items():
        if only_sizes and name not in only_sizes:
            continue
        entry = {"shape": s}
        sc, fc = sanevik_config(s), felolorn_config(s)
        for label, cfg, wb, runs in (("sanevik", sc, sanevik_decode_weight_bytes(sc, batch), s["layers"] + 2),
                                     ("gazutar", gazutar_config(s), decode_weight_bytes(s, batch, True), s["layers"]),
                                     ("felolorn", fc, felolorn_decode_weight_bytes(fc, batch), s["layers"]),
                                     ("qwen3_moe", qwen3_moe_config(s), decode_weight_bytes(s, batch, False), s["layers"])):
            if label not in only_models:
                continue
            r = run_model(cfg, batch, prompt_len, args.steps, args.warmup)
            r["layer_runs"] = runs
            r["decode_weight_bytes"] = wb
            r["decode_weight_roofline_frac"] = wb / (r["ms_per_decode_step"] * 1e-3) / HBM_BYTES_PER_S
            entry[label] = r
        for other in ("gazutar", "felolorn"):
            if "sanevik" in entry and other in entry:
                entry["sanevik_vs_" + other] = {k: entry["sanevik"][k] / entry[other][k] for k in ("prefill_tok_s", "decode_tok_s")}
                entry["sanevik_vs_" + other + "_per_layer_run"] = {
                    k: v * entry["sanevik"]["layer_runs"] / entry[other]["layer_runs"] for k, v in entry["sanevik_vs_" + other].items()}
        out["sizes"][name] = entry
    print(json.dumps(out), flush=True)
    return out
