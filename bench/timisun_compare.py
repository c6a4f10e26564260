"""Prefill and decode throughput of the Timisun design beside the closest uniform family (Llama: RMS norm, gated
feed-forward) at equal size, random weights, through the serving engine (scheduler, paged cache, decode graphs,
sampler). Run as ``python bench.py --timisun [SIZE,...]``.

"Equal size": same width, layer count, head count and vocabulary; the dense model's feed-forward width equals the
feed-forward rows a Timisun token touches (top * expert ff + shared ff), its heads are 128 wide and all of them
are cached (the latent cache holds one row of kv_rank numbers per token and layer instead).
"""
from __future__ import annotations

import time

import numpy as np
import torch

SIZES = {
    # name: width, layers, heads, dim, vdim, kv_rank, window, experts, top, ff, shared ff, vocab
    "w2048": dict(width=2048, layers=4, heads=16, dim=128, vdim=128, rank=256, window=1024, experts=32, top=4, ff=768,
                  shared=1024, vocab=32000),
    "w4096": dict(width=4096, layers=2, heads=32, dim=128, vdim=128, rank=256, window=2048, experts=64, top=4, ff=1536,
                  shared=2048, vocab=32000),
    "w1024": dict(width=1024, layers=4, heads=8, dim=64, vdim=64, rank=128, window=512, experts=16, top=2, ff=512,
                  shared=1024, vocab=32000),
}


def timisun_dict(s):
    mixer = dict(heads=s["heads"], dim=s["dim"], vdim=s["vdim"], kv_rank=s["rank"], scale=s["dim"] ** -0.5,
                 mask=dict(size=s["window"]))
    mlp = dict(kind="moe", router=dict(experts=s["experts"], top=s["top"]), expert=dict(ff=s["ff"], limit=7.0),
               shared=dict(ff=s["shared"], limit=7.0))
    layers = []
    for i in range(s["layers"]):
        m = dict(mixer)
        if i % 2 == 1:
            m["kv_from"] = i - 1  # every second layer reads its neighbour's latent rows
        layers.append(dict(type="latent_attention", mixer=m, mlp=mlp))
    return dict(architecture="Timisun", vocab=s["vocab"], width=s["width"], embedding=dict(scale=1.0),
                norm=dict(eps=1e-6), layers=layers)


def build(kind, s, dev):
    from llmss_amd.models.config import ModelConfig, get_preset
    from llmss_amd.models.layered import create_model
    from llmss_amd.models.weights import random_timisun_weights, random_weights

    if kind == "timisun":
        cfg = ModelConfig.from_hf_dict(timisun_dict(s))
        return create_model(cfg, random_timisun_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))
    cfg = get_preset("llama2-7b", hidden_size=s["width"], num_layers=s["layers"], num_heads=s["heads"],
                     num_kv_heads=s["heads"], head_dim=s["width"] // s["heads"],
                     intermediate_size=s["top"] * s["ff"] + s["shared"], vocab_size=s["vocab"],
                     max_position_embeddings=8192, rotary_dim=s["width"] // s["heads"])
    return create_model(cfg, random_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))


def measure(model, batch, prompt_len, gen_len, rounds, progress):
    from llmss_amd.engine import LLMEngine, SamplingParams

    eng = LLMEngine(model, max_num_seqs=batch, max_batched_tokens=max(8192, prompt_len), block_size=16,
                    max_model_len=prompt_len + gen_len + 16)
    rng = np.random.default_rng(3)
    V = model.cfg.vocab_size
    sp = SamplingParams(max_new_tokens=gen_len, temperature=1.0, top_p=0.95, top_k=50, ignore_eos=True, seed=5)
    out = None
    for r in range(rounds + 1):  # round 0 warms up
        for k in ("prefill_time_s", "decode_time_s"):
            eng.stats[k] = 0.0
        for k in ("prefill_tokens", "decode_steps", "tokens"):
            eng.stats[k] = 0
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        eng.generate([rng.integers(0, V, prompt_len).tolist() for _ in range(batch)], sp)
        torch.cuda.synchronize()
        el = time.perf_counter() - t0
        st = eng.stats
        res = dict(prefill_tok_s=st["prefill_tokens"] / max(st["prefill_time_s"], 1e-9),
                   decode_tok_s=(st["tokens"] - batch) / max(st["decode_time_s"], 1e-9),
                   decode_ms_per_step=1e3 * st["decode_time_s"] / max(st["decode_steps"], 1), total_s=el)
        progress(f"  round {r}: " + ", ".join(f"{k} {v:.1f}" for k, v in res.items()))
        if r and (out is None or res["total_s"] < out["total_s"]):
            out = res
    del eng
    torch.cuda.empty_cache()
    return {k: round(v, 2) for k, v in out.items()}


def run(sizes, batch, prompt_len, gen_len, rounds, progress, kinds=("timisun", "dense")):
    dev = torch.device("cuda", torch.cuda.current_device())
    rows = []
    for name in sizes:
        s = SIZES[name]
        row = dict(size=name, shape=s, batch=batch, prompt_len=prompt_len, gen_len=gen_len)
        for kind in kinds:
            progress(f"{name} {kind}: building")
            model = build(kind, s, dev)
            row[kind] = measure(model, batch, prompt_len, gen_len, rounds, progress)
            row[kind]["params_M"] = round(model.cfg.num_params() / 1e6, 1)
            del model
            torch.cuda.empty_cache()
        if "timisun" in row and "dense" in row:
            row["prefill_ratio"] = round(row["timisun"]["prefill_tok_s"] / row["dense"]["prefill_tok_s"], 3)
            row["decode_ratio"] = round(row["timisun"]["decode_tok_s"] / row["dense"]["decode_tok_s"], 3)
        rows.append(row)
    return dict(metric="timisun_vs_dense_tokens_per_sec", unit="tokens/s", dtype="bf16", data="synthetic",
                sizes=rows)
