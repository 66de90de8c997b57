"""Prefill and decode throughput of the layer-list designs (Nibalix,
Nedasun, Kakilorn, Legilix) beside one another and beside the dense transformer of equal size
(``bench.py --hybrid-bench``).

All models get random weights at layer sizes that resemble a real model
and run through their own engine's ``generate`` — scheduler, cache, step
function and sampler included. Prefill tokens/s is timed with one output
token per prompt; decode tokens/s from the extra time of a longer
generation.
"""

from __future__ import annotations

import gc
import json
import time

import torch

from .config import EngineConfig, SamplingParams

# name -> sizes. The dense twin has the same width, depth, head count and
# head size, and an MLP as wide as the experts one token uses.
SIZES = {
    "1k": dict(width=1024, layers=8, heads=8, dim=64, rot_dim=64, vdim=128,
               kv_rank=256, window=512, experts=8, top=2, ff=512, vocab=32000),
    "2k": dict(width=2048, layers=8, heads=16, dim=64, rot_dim=64, vdim=128,
               kv_rank=512, window=1024, experts=8, top=2, ff=1024, vocab=32000),
}


def nibalix_bench_config(s: dict) -> dict:
    """Layer pattern: latent attention, latent attention, latent attention
    reading the previous layer's cache, minGRU."""
    moe = {"kind": "moe", "expert": {"ff": s["ff"]},
           "router": {"experts": s["experts"], "top": s["top"]}}
    layers = []
    for i in range(s["layers"]):
        if i % 4 == 3:
            layers.append({"type": "mingru", "mixer": {"width": s["width"]}, "mlp": moe})
            continue
        mc = {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot_dim"],
              "vdim": s["vdim"], "kv_rank": s["kv_rank"],
              "scale": (s["dim"] + s["rot_dim"]) ** -0.5,
              "rot": {"base": 10000.0, "dims": s["rot_dim"]},
              "mask": {"size": s["window"]}}
        if i % 4 == 2:
            mc["kv_from"] = i - 1
        layers.append({"type": "latent_attention", "mixer": mc, "mlp": moe})
    return {"architecture": "Nibalix", "canon": {"taps": 4}, "layers": layers,
            "norm": {"eps": 1e-5}, "residual_mult": 0.5, "vocab": s["vocab"],
            "width": s["width"]}


def nedasun_bench_config(s: dict) -> dict:
    """Same width, depth, head count and expert sizes as the Nibalix config
    of the size: attention and delta-rule layers alternate (every fourth
    layer pair starts with a dense feed-forward), 4 query heads per kv
    head, one identity expert and a shared expert as wide as one expert."""
    kvh = max(1, s["heads"] // 4)
    moe = {"kind": "moe", "expert": {"ff": s["ff"], "limit": 7.0},
           "router": {"experts": s["experts"], "identity": 1, "scale": 1.0,
                      "top": s["top"]},
           "shared": {"ff": s["ff"], "limit": 7.0}}
    dense = {"kind": "dense", "ff": s["top"] * s["ff"], "limit": 7.0}
    layers = []
    for i in range(s["layers"]):
        mlp = dense if i == 0 else moe
        if i % 2 == 0:
            mc = {"heads": s["heads"], "kv_heads": kvh, "dim": 128, "vdim": 128,
                  "scale": 128 ** -0.5, "softcap": 30.0, "v_mix": True,
                  "rot": {"base": 10000.0, "dims": 64}}
            layers.append({"type": "attention", "mixer": mc, "mlp": mlp})
        else:
            mc = {"heads": s["heads"], "kv_heads": kvh, "dim": 128, "vdim": 128,
                  "conv": 4}
            layers.append({"type": "delta", "mixer": mc, "mlp": mlp})
    return {"architecture": "Nedasun", "layers": layers, "norm": {"eps": 1e-5},
            "vocab": s["vocab"], "width": s["width"]}


def kakilorn_bench_config(s: dict) -> dict:
    """Same width, depth and head count as the other designs of the size,
    head sizes of the Nedasun config (128/128, 4 query heads per kv head)
    and the latent sizes of the Nibalix config. Layer pattern: channel-decay
    delta rule, latent attention, latent attention, sigmoid attention beside
    the per-head delta rule; dense feed-forwards as wide as the experts one
    token uses elsewhere (none after the first layer of each group)."""
    kvh = max(1, s["heads"] // 4)
    dense = {"kind": "dense", "ff": s["top"] * s["ff"]}
    delta = {"heads": s["heads"], "kv_heads": kvh, "dim": 128, "vdim": 128, "conv": 4}
    layers = []
    for i in range(s["layers"]):
        if i % 4 == 0:
            mc = dict(delta, decay_rank=s["width"] // 16, gate_rank=s["width"] // 16)
            layers.append({"type": "channel_delta", "mixer": mc, "mlp": None})
        elif i % 4 == 3:
            left = {"heads": s["heads"], "kv_heads": kvh, "dim": 128, "vdim": 128,
                    "scale": 128 ** -0.5,
                    "mask": {"size": s["window"], "keep_first": 16}}
            mc = {"left": left, "right": dict(delta, heads=s["heads"] // 2,
                                              kv_heads=max(1, kvh // 2)),
                  "left_scale": 1.0, "right_scale": 1.0}
            layers.append({"type": "parallel", "mixer": mc, "mlp": dense})
        else:
            mc = {"heads": s["heads"], "dim": s["dim"], "rot_dim": s["rot_dim"],
                  "vdim": s["vdim"], "kv_rank": s["kv_rank"],
                  "q_rank": s["kv_rank"] * 3 // 2,
                  "scale": (s["dim"] + s["rot_dim"]) ** -0.5,
                  "rot": {"base": 10000.0, "dims": s["rot_dim"],
                          "scaling": {"factor": 4.0, "original": 4096,
                                      "fast": 32.0, "slow": 1.0}}}
            layers.append({"type": "latent_attention", "mixer": mc, "mlp": dense})
    return {"architecture": "Kakilorn", "embedding": {"scale": 1.0},
            "layers": layers, "logit_scale": 1.0, "norm": {"eps": 1e-5},
            "vocab": s["vocab"], "width": s["width"]}


def legilix_bench_config(s: dict) -> dict:
    """Same width, depth, head count and head sizes (128/128, 4 query heads
    per kv head) as the Nedasun config of the size; every layer is windowed
    attention: the distance-bias form and the rotary form with mixed scores
    alternate (window of the size, 16 kept tokens), feed-forwards alternate
    between the experts of the other designs and a dense MLP as wide as the
    experts one token uses; norms over four groups."""
    kvh = max(1, s["heads"] // 4)
    moe = {"kind": "moe", "expert": {"ff": s["ff"]},
           "router": {"experts": s["experts"], "top": s["top"]}}
    dense = {"kind": "dense", "ff": s["top"] * s["ff"]}
    base = {"heads": s["heads"], "kv_heads": kvh, "dim": 128, "vdim": 128,
            "scale": 128 ** -0.5}
    layers = []
    for i in range(s["layers"]):
        if i % 2 == 0:
            mc = dict(base, mask={"size": s["window"]})
            layers.append({"type": "attention_2", "mixer": mc,
                           "mlp": dense if i % 4 == 0 else moe})
        else:
            mc = dict(base, mask={"size": s["window"], "keep_first": 16},
                      rot={"base": 10000.0, "dims": 64,
                           "scaling": {"factor": 4.0, "original": 4096,
                                       "fast": 32.0, "slow": 1.0}})
            layers.append({"type": "attention", "mixer": mc,
                           "mlp": moe if i % 4 == 1 else dense})
    return {"architecture": "Legilix", "embedding": {"scale": 1.0},
            "layers": layers, "logit_scale": 1.0,
            "norm": {"eps": 1e-5, "groups": 4}, "vocab": s["vocab"],
            "width": s["width"]}


def _build_hybrid(s, device, max_len, batch, design="nibalix"):
    from .engine.hybrid_engine import HybridEngine
    from .models.hybrid import (HybridLM, kakilorn_spec_from_config,
                                legilix_spec_from_config,
                                nedasun_spec_from_config,
                                nibalix_spec_from_config)
    if design == "legilix":
        spec = legilix_spec_from_config(legilix_bench_config(s))
    elif design == "kakilorn":
        spec = kakilorn_spec_from_config(kakilorn_bench_config(s))
    elif design == "nedasun":
        spec = nedasun_spec_from_config(nedasun_bench_config(s))
    else:
        spec = nibalix_spec_from_config(nibalix_bench_config(s))
    model = HybridLM(spec, dtype=torch.bfloat16, device=device).random_init(1)
    cfg = EngineConfig(max_seq_length=max_len, kv_block_size=16,
                       num_kv_blocks=batch * ((max_len + 15) // 16) + 8,
                       num_state_slots=batch, max_num_seqs=batch,
                       step_token_budget=8192)
    return HybridEngine(model, cfg, device=device)


def _build_dense(s, device, max_len, batch):
    from .engine.engine import Engine
    from .models.model import CausalLM
    from .models.spec import ModelSpec
    spec = ModelSpec(f"dense-{s['width']}", s["vocab"], s["width"],
                     s["top"] * s["ff"], s["layers"], s["heads"], s["heads"],
                     128, 1e4, 1e-5, False, False, max_position=max_len)
    model = CausalLM(spec, dtype=torch.bfloat16, device=device).random_init(1)
    cfg = EngineConfig(max_seq_length=max_len, kv_block_size=16,
                       num_kv_blocks=batch * ((max_len + 15) // 16) + 8,
                       max_num_seqs=batch)
    return Engine(model, cfg, device=device)


def _timed(engine, prompts, new_tokens, device):
    sp = SamplingParams(max_tokens=new_tokens, temperature=1.0, n=1)
    if device.type == "cuda":
        torch.cuda.synchronize()
    t0 = time.perf_counter()
    engine.generate(prompts, sp, eos_token_id=None)
    if device.type == "cuda":
        torch.cuda.synchronize()
    return time.perf_counter() - t0


def measure(engine, vocab, batch, prompt_len, new_tokens, device):
    g = torch.Generator().manual_seed(0)
    prompts = torch.randint(0, vocab, (batch, prompt_len), generator=g).tolist()
    _timed(engine, prompts[:2], 4, device)                 # warm-up
    _timed(engine, prompts, new_tokens, device)            # graphs, allocator
    t_pre = min(_timed(engine, prompts, 1, device) for _ in range(2))
    t_all = min(_timed(engine, prompts, new_tokens, device) for _ in range(2))
    dec = max(t_all - t_pre, 1e-9)
    return {"prefill_tok_s": batch * prompt_len / t_pre,
            "decode_tok_s": batch * (new_tokens - 1) / dec,
            "prefill_s": t_pre, "decode_ms_per_step": 1e3 * dec / (new_tokens - 1)}


def run(sizes, device, batch=16, prompt_len=1024, new_tokens=33, which=("legilix", "kakilorn", "nedasun", "nibalix", "dense")):
    out = []
    for name in sizes:
        s = SIZES[name]
        max_len = prompt_len + new_tokens + 1
        for kind in which:
            if kind == "dense":
                eng = _build_dense(s, device, max_len, batch)
            else:
                eng = _build_hybrid(s, device, max_len, batch, design=kind)
            r = measure(eng, s["vocab"], batch, prompt_len, new_tokens, device)
            line = {"bench": "hybrid", "size": name, "model": kind, "batch": batch,
                    "prompt_len": prompt_len, "new_tokens": new_tokens, "dtype": "bf16",
                    "data": "synthetic", **{k: round(v, 3) for k, v in r.items()}}
            print(json.dumps(line), flush=True)
            out.append(line)
            del eng
            gc.collect()        # the engine and its captured steps are a cycle
            if device.type == "cuda":
                torch.cuda.empty_cache()
    return out
