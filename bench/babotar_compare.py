"""Prefill and decode throughput of the Babotar design beside the closest uniform family (Llama: pre-norm sequential
blocks, rotary grouped-query attention, gated feed-forward) at equal size, random weights, through the serving engine
(scheduler, paged cache, state slots, decode graphs, sampler). Run as ``python bench.py --babotar [SIZE,...]``.

"Equal size": same width, layer count, vocabulary and feed-forward width; the dense model's attention has the heads,
key/value heads and head size of Babotar's attention branch. Babotar's layers follow the pattern parallel, parallel,
decay, parallel (repeated), with two residual streams and a four-tap input convolution.
"""
from __future__ import annotations

import torch

from timisun_compare import measure

SIZES = {
    # width, layers, attention heads / kv heads / head size, rotated dims, delta-rule heads / key heads / key / value
    # size, decay heads / key / value size, feed-forward, vocab
    "w1024": dict(width=1024, layers=4, heads=8, kv=2, dim=128, rot=64, dheads=8, dkv=4, ddim=64, dvdim=128,
                  lheads=8, ldim=128, lvdim=128, ff=2816, vocab=32000),
    "w2048": dict(width=2048, layers=4, heads=16, kv=4, dim=128, rot=64, dheads=16, dkv=8, ddim=128, dvdim=128,
                  lheads=16, ldim=128, lvdim=128, ff=5632, vocab=32000),
    "w4096": dict(width=4096, layers=3, heads=32, kv=8, dim=128, rot=64, dheads=32, dkv=16, ddim=128, dvdim=128,
                  lheads=32, ldim=128, lvdim=128, ff=11008, vocab=32000),
}


def babotar_dict(s, max_positions=8192):
    par = dict(type="parallel", mlp=dict(kind="dense", ff=s["ff"]), mixer=dict(
        left=dict(heads=s["heads"], kv_heads=s["kv"], dim=s["dim"], vdim=s["dim"], scale=s["dim"] ** -0.5, softcap=30.0,
                  rot=dict(base=10000.0, dims=s["rot"], scaling=dict(factor=4.0, original=4096, fast=16.0, slow=2.0))),
        right=dict(heads=s["dheads"], kv_heads=s["dkv"], dim=s["ddim"], vdim=s["dvdim"], conv=4),
        left_scale=1.0, right_scale=1.0))
    lig = dict(type="lightning", mlp=dict(kind="dense", ff=s["ff"]), mixer=dict(
        heads=s["lheads"], dim=s["ldim"], vdim=s["lvdim"],
        decay=[1.0 - 2.0 ** (-3 - 5 * i / max(1, s["lheads"] - 1)) for i in range(s["lheads"])]))
    layers = [lig if i % 4 == 2 else par for i in range(s["layers"])]
    return dict(architecture="Babotar", vocab=s["vocab"], width=s["width"], max_positions=max_positions,
                norm=dict(eps=1e-6), residual_mult=1.0, streams=2, canon=dict(taps=4), layers=layers)


def build(kind, s, dev):
    from llmss_amd.models.config import ModelConfig, get_preset
    from llmss_amd.models.layered import create_model
    from llmss_amd.models.weights import random_babotar_weights, random_weights

    if kind == "babotar":
        cfg = ModelConfig.from_hf_dict(babotar_dict(s))
        return create_model(cfg, random_babotar_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))
    cfg = get_preset("llama2-7b", hidden_size=s["width"], num_layers=s["layers"], num_heads=s["heads"],
                     num_kv_heads=s["kv"], head_dim=s["dim"], intermediate_size=s["ff"], vocab_size=s["vocab"],
                     max_position_embeddings=8192, rotary_dim=s["dim"])
    return create_model(cfg, random_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))


def run(sizes, batch, prompt_len, gen_len, rounds, progress, kinds=("babotar", "dense")):
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
        if "babotar" in row and "dense" in row:
            row["prefill_ratio"] = round(row["babotar"]["prefill_tok_s"] / row["dense"]["prefill_tok_s"], 3)
            row["decode_ratio"] = round(row["babotar"]["decode_tok_s"] / row["dense"]["decode_tok_s"], 3)
        rows.append(row)
    return dict(metric="babotar_vs_dense_tokens_per_sec", unit="tokens/s", dtype="bf16", data="synthetic",
                sizes=rows)
