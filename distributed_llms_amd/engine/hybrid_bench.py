"""Prefill and decode throughput of a layer-list model beside the closest flat-config model of equal
size (``bench.py --hybrid``), random weights, one GPU: Tudilix (sliding-window attention + RG-LRU) beside
a Llama-architecture model of the same width, layer count, feed-forward size, head size and K/V heads;
Gikovik (latent attention + grouped-choice mixture of experts) beside a Mixtral-architecture model of the
same width, layer count, heads, expert count and experts per token, with expert weights of equal size;
Zebutar (chunked attention beside a gated delta rule, SwiGLU experts) beside the same Mixtral model;
Fekizen (window attention with averaged blocks beside gated linear attention, lightning layers, SwiGLU experts)
beside the same Mixtral model and, for its kernels, beside Zebutar.  Every step goes through the engine's StageRunner (the trace
replayer builds the batches): one step with ``batch`` prompts of ``prompt_len`` tokens (prefill),
then ``gen_len`` steps of one token per sequence (decode)."""
from __future__ import annotations

import json
import time

import numpy as np
import torch

from ..config import EngineConfig, ModelConfig
from ..models import make_stage
from .llm_engine import LLMEngine
from .replay import TraceReplayer

# name -> (width, layers, ff, heads, kv_heads, head size, rglru blocks, window)
SIZES = {
    "2b": (2560, 6, 7680, 16, 4, 128, 10, 2048),
    "9b": (4096, 6, 12288, 32, 8, 128, 16, 2048),
    "small": (1024, 6, 3072, 8, 2, 128, 4, 512),
}


def hybrid_config(size: str, vocab: int = 32000) -> ModelConfig:
    w, nl, ff, h, g, d, nb, win = SIZES[size]
    rot = {"base": 10000.0, "dims": d // 2, "scaling": {"factor": 4.0, "fast": 32.0, "original": 4096, "slow": 1.0}}
    layers = []
    for i in range(nl):
        mlp = {"kind": "dense", "ff": ff, "limit": 7.0}
        if i % 3 == 2:
            layers.append({"type": "attention", "mlp": mlp, "mixer": {
                "conv": 4, "dim": d, "vdim": d, "heads": h, "kv_heads": g, "mask": {"size": win},
                "scale": d ** -0.5, "rot": rot}})
        else:
            layers.append({"type": "rglru", "mlp": mlp, "mixer": {"blocks": nb, "conv": 4, "width": w}})
    return ModelConfig.from_hf_config({"architecture": "Tudilix", "vocab": vocab, "width": w, "residual_mult": 1.0,
                                       "logit_softcap": 30.0, "norm": {"eps": 1e-6}, "layers": layers},
                                      name=f"tudilix-{size}")


def llama_config(size: str, vocab: int = 32000) -> ModelConfig:
    w, nl, ff, h, g, d, _nb, _win = SIZES[size]
    return ModelConfig(name=f"llama-{size}", arch="llama", vocab_size=vocab, hidden_size=w, intermediate_size=ff,
                       num_layers=nl, num_heads=h, num_kv_heads=g, head_dim=d, max_position=8192)


# name -> (width, layers, dense ff, heads, dim, rot_dim, vdim, kv_rank, q_rank, experts, top, expert ff)
GIKOVIK_SIZES = {
    "small": (1024, 6, 3072, 8, 64, 32, 64, 128, 384, 8, 2, 1024),
    "2b": (2560, 6, 7680, 16, 128, 64, 128, 192, 768, 8, 2, 2560),
    "9b": (4096, 6, 12288, 32, 128, 64, 128, 192, 1536, 8, 2, 4096),
}


def gikovik_config(size: str, vocab: int = 32000) -> ModelConfig:
    """Layers 0 and 3 dense, the others mixtures with a shared expert; every third layer the sink form,
    the others the rotated form; the first three layers as a loop that runs once (its entry projection
    is part of the step); a 64-column token input."""
    w, nl, ff, h, d, dr, dv, r, qr, e, top, ef = GIKOVIK_SIZES[size]
    moe = {"kind": "moe", "expert": {"ff": ef}, "shared": {"ff": ef},
           "router": {"experts": e, "groups": {"count": 4, "keep": 2}, "scale": 2.5, "top": top}}
    layers = []
    for i in range(nl):
        m = {"heads": h, "dim": d, "vdim": dv, "kv_rank": r + (dr if i % 3 == 2 else 0), "q_rank": qr,
             "scale": (d + dr) ** -0.5}
        kind = "latent_attention"
        if i % 3 != 2:
            kind = "latent_attention_2"
            m.update({"rot_dim": dr, "rot": {"base": 10000.0, "dims": dr}})
        layers.append({"type": kind, "mixer": m, "mlp": {"kind": "dense", "ff": ff} if i % 3 == 0 else moe})
    return ModelConfig.from_hf_config({"architecture": "Gikovik", "vocab": vocab, "width": w, "norm": {"eps": 1e-6},
                                       "token_side": {"dim": 64}, "loop": {"start": 0, "stop": 3, "times": 1},
                                       "layers": layers}, name=f"gikovik-{size}")


def mixtral_config(size: str, vocab: int = 32000) -> ModelConfig:
    """Same width, layers, heads, experts and experts per token; three-matrix SwiGLU experts of 2/3 the
    width of the two-matrix ones (rounded up to 256), i.e. expert weights of equal size."""
    w, nl, _ff, h, _d, _dr, _dv, _r, _qr, e, top, ef = GIKOVIK_SIZES[size]
    inter = -(-(2 * ef // 3) // 256) * 256
    return ModelConfig(name=f"mixtral-{size}", arch="mixtral", vocab_size=vocab, hidden_size=w, intermediate_size=inter,
                       num_layers=nl, num_heads=h, num_kv_heads=max(1, h // 4), head_dim=128, max_position=8192,
                       rope_theta=1000000.0, num_experts=e, experts_per_token=top)


def zebutar_config(size: str, vocab: int = 32000) -> ModelConfig:
    """Width, layers, heads, experts and experts per token of the Gikovik / Mixtral sizes; attention with the
    Mixtral model's heads (a quarter as many K/V heads, 128-wide, half of every head rotated) inside chunks
    of 2048 positions, beside a delta rule with as many 128 x 128 states as attention heads and half as many
    q / k heads, 4-tap convolutions; layers 0 and 3 dense, the others mixtures of three-matrix experts of the
    Mixtral model's size with a shared expert."""
    w, nl, ff, h, _d, _dr, _dv, _r, _qr, e, top, ef = GIKOVIK_SIZES[size]
    inter = -(-(2 * ef // 3) // 256) * 256
    moe = {"kind": "moe", "expert": {"ff": inter}, "shared": {"ff": inter}, "router": {"experts": e, "top": top}}
    mixer = {"left": {"heads": h, "kv_heads": max(1, h // 4), "dim": 128, "vdim": 128, "mask": {"size": 2048},
                      "scale": 128 ** -0.5, "rot": {"base": 10000.0, "dims": 64}},
             "right": {"heads": h, "kv_heads": max(1, h // 2), "dim": 128, "vdim": 128, "conv": 4},
             "left_scale": 1.0, "right_scale": 1.0}
    layers = [{"type": "parallel", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if i % 3 == 0 else moe}
              for i in range(nl)]
    return ModelConfig.from_hf_config({"architecture": "Zebutar", "vocab": vocab, "width": w, "norm": {"eps": 1e-6},
                                       "layers": layers}, name=f"zebutar-{size}")


def fekizen_config(size: str, vocab: int = 32000) -> ModelConfig:
    """Width, layers, heads, experts and experts per token of the Gikovik / Mixtral sizes.  Odd layers are
    parallel: attention with the Mixtral model's heads (a quarter as many K/V heads, 128-wide, half of every
    head rotated with blended frequencies, a window of 1024 positions plus one averaged key per 16 older
    positions, capped scores, sinks) beside gated linear attention with as many 128 x 128 states as attention
    heads; even layers are lightning attention with the same states.  Every layer has a mixture of three-matrix
    experts of the Mixtral model's size with a shared expert; the first two layers are a loop that runs once
    (its entry is part of the step)."""
    w, nl, _ff, h, _d, _dr, _dv, _r, _qr, e, top, ef = GIKOVIK_SIZES[size]
    inter = -(-(2 * ef // 3) // 256) * 256
    moe = {"kind": "moe", "expert": {"ff": inter}, "shared": {"ff": inter}, "router": {"experts": e, "top": top}}
    par = {"left": {"heads": h, "kv_heads": max(1, h // 4), "dim": 128, "vdim": 128, "mask": {"size": 1024, "pool": 16},
                    "scale": 128 ** -0.5, "softcap": 30.0,
                    "rot": {"base": 10000.0, "dims": 64,
                            "scaling": {"factor": 4.0, "fast": 32.0, "original": 4096, "slow": 1.0}}},
           "right": {"heads": h, "dim": 128, "vdim": 128, "tau": 8.0, "rank": 32}}
    light = {"heads": h, "dim": 128, "vdim": 128, "decay": [1.0 - 2.0 ** -(3.0 + 6.0 * i / h) for i in range(h)]}
    layers = [{"type": "parallel", "mixer": par, "mlp": moe} if i % 2 else {"type": "lightning", "mixer": light, "mlp": moe}
              for i in range(nl)]
    return ModelConfig.from_hf_config({"architecture": "Fekizen", "vocab": vocab, "width": w, "norm": {"eps": 1e-6},
                                       "embedding": {"scale": float(w) ** 0.5}, "max_positions": 8192,
                                       "loop": {"start": 0, "stop": 2, "times": 1}, "layers": layers},
                                      name=f"fekizen-{size}")


def _measure(mcfg: ModelConfig, batch: int, prompt_len: int, gen_len: int, reps: int, tmp: str, graphs: bool):
    import os
    os.makedirs(tmp, exist_ok=True)
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(mcfg.to_hf_config(), f)
    stage = make_stage(mcfg, device="cuda", dtype=torch.bfloat16).init_synthetic(0)
    total = batch * (prompt_len + gen_len + 32)
    ecfg = EngineConfig(model=tmp, shard_dir=tmp, device="cuda", dtype="bfloat16", max_batch=batch,
                        max_seq_len=prompt_len + gen_len + 8, kv_block_size=32,
                        num_kv_blocks=-(-total // 32) + batch + 2, max_prefill_tokens=batch * prompt_len,
                        use_graphs=graphs, graph_batch_sizes=(batch,))
    eng = LLMEngine(ecfg, stage)
    rp = TraceReplayer(eng)
    rng = np.random.default_rng(0)
    pre, dec = [], []
    for r in range(reps + 1):
        names = [f"q{r}_{i}" for i in range(batch)]
        toks = rng.integers(10, mcfg.vocab_size - 1, size=(batch, prompt_len + gen_len)).tolist()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        rp.step([(n, toks[i][:prompt_len], [prompt_len - 1]) for i, n in enumerate(names)])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for k in range(gen_len):
            rp.step([(n, [toks[i][prompt_len + k]], [0]) for i, n in enumerate(names)],
                    end=names if k == gen_len - 1 else ())
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        if r:                   # the first round warms up (allocations, graph capture)
            pre.append(t1 - t0)
            dec.append(t2 - t1)
    del eng, rp, stage
    torch.cuda.empty_cache()
    return batch * prompt_len / min(pre), batch * gen_len / min(dec)


MAKERS = {"tudilix": hybrid_config, "llama": llama_config, "gikovik": gikovik_config, "mixtral": mixtral_config,
          "zebutar": zebutar_config, "fekizen": fekizen_config}
PAIRS = {"tudilix": "llama", "gikovik": "mixtral", "zebutar": "mixtral", "fekizen": "mixtral"}


def run(size: str = "2b", batch: int = 32, prompt_len: int = 1024, gen_len: int = 32, reps: int = 2,
        tmp: str = "/tmp/dllm_hybrid_bench", models=("tudilix", "llama")) -> dict:
    """``models``: which to run, of tudilix, llama, gikovik, zebutar, fekizen, mixtral; a layer-list model and its
    flat counterpart (tudilix / llama, gikovik / mixtral, zebutar / mixtral, fekizen / mixtral) also get the ratio
    of their throughputs (``ratios`` holds every pair that ran; ``prefill_ratio`` / ``decode_ratio`` the first)."""
    out = {"size": size, "batch": batch, "prompt_len": prompt_len, "gen_len": gen_len, "dtype": "bf16",
           "data": "synthetic (random-init weights, random token ids)"}
    for key in models:
        cfg = MAKERS[key](size)
        p, d = _measure(cfg, batch, prompt_len, gen_len, reps, f"{tmp}/{key}", True)
        out[key] = {"prefill_tok_s": round(p, 1), "decode_tok_s": round(d, 1),
                    "params_m": round(cfg.param_count() / 1e6, 1)}
    for a, b in PAIRS.items():
        if a in out and b in out:
            pr = round(out[a]["prefill_tok_s"] / out[b]["prefill_tok_s"], 3)
            dr = round(out[a]["decode_tok_s"] / out[b]["decode_tok_s"], 3)
            out.setdefault("ratios", {})[f"{a}/{b}"] = {"prefill": pr, "decode": dr}
            out.setdefault("prefill_ratio", pr)
            out.setdefault("decode_ratio", dr)
    return out
