"""Prefill and decode throughput of the Lamisun design beside the closest uniform family (Llama: sequential blocks,
RMS norm, rotary grouped-query attention, dense feed-forward) at equal size, random weights, through the serving
engine (scheduler, paged cache, state slots, decode graphs, sampler). Run as ``python bench.py --lamisun [SIZE,...]``.

"Equal size": same width, layer count and vocabulary; the dense model's attention has the heads, key/value heads of
Lamisun's two-map attention and twice its key size (two maps of ``dim`` are one head of 2 ``dim``); its gated
feed-forward holds as many weights as Lamisun's plain one (ff x 2 / 3). Lamisun's layers alternate latent attention
and two-map attention, every layer with a feed-forward, four-tap input convolutions before both sublayers.
"""
from __future__ import annotations

import torch

from timisun_compare import measure

SIZES = {
    # width, layers; latent attention: heads / plain key size / rotated size / value size / latent rank (rank + rotated
    # size = the cached row); two-map attention: heads / key heads / key size per map / value size / chunk; feed-forward
    "w1024": dict(width=1024, layers=4, lheads=8, ldim=64, lrot=64, lvdim=128, rank=192, heads=8, kv=2, dim=64,
                  vdim=128, chunk=512, ff=4224, vocab=32000, buckets=16381),
    "w2048": dict(width=2048, layers=4, lheads=16, ldim=128, lrot=64, lvdim=128, rank=192, heads=16, kv=4, dim=64,
                  vdim=128, chunk=1024, ff=8448, vocab=32000, buckets=16381),
    "w4096": dict(width=4096, layers=2, lheads=32, ldim=128, lrot=64, lvdim=128, rank=192, heads=32, kv=8, dim=64,
                  vdim=128, chunk=2048, ff=16512, vocab=32000, buckets=16381),
}


def lamisun_dict(s):
    mlp = dict(kind="dense", ff=s["ff"])
    lat = dict(type="latent_attention", mlp=mlp, mixer=dict(
        heads=s["lheads"], dim=s["ldim"], rot_dim=s["lrot"], vdim=s["lvdim"], kv_rank=s["rank"],
        scale=(s["ldim"] + s["lrot"]) ** -0.5, rot=dict(base=10000.0, dims=s["lrot"])))
    att = dict(type="attention", mlp=mlp, mixer=dict(
        heads=s["heads"], kv_heads=s["kv"], dim=s["dim"], vdim=s["vdim"], scale=s["dim"] ** -0.5, diff=0.3,
        mask=dict(size=s["chunk"])))
    return dict(architecture="Lamisun", vocab=s["vocab"], width=s["width"], norm=dict(eps=1e-6), canon=dict(taps=4),
                embedding=dict(scale=1.0, bigram=dict(buckets=s["buckets"], mul_prev=1000003, mul_cur=7919)),
                layers=[lat if i % 2 == 0 else att for i in range(s["layers"])])


def build(kind, s, dev):
    from llmss_amd.models.config import ModelConfig, get_preset
    from llmss_amd.models.layered import create_model
    from llmss_amd.models.weights import random_lamisun_weights, random_weights

    if kind == "lamisun":
        cfg = ModelConfig.from_hf_dict(lamisun_dict(s))
        return create_model(cfg, random_lamisun_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))
    cfg = get_preset("llama2-7b", hidden_size=s["width"], num_layers=s["layers"], num_heads=s["heads"],
                     num_kv_heads=s["kv"], head_dim=2 * s["dim"], intermediate_size=s["ff"] * 2 // 3 // 64 * 64,
                     vocab_size=s["vocab"], max_position_embeddings=8192, rotary_dim=2 * s["dim"])
    return create_model(cfg, random_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))


def run(sizes, batch, prompt_len, gen_len, rounds, progress, kinds=("lamisun", "dense")):
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
        if "lamisun" in row and "dense" in row:
            row["prefill_ratio"] = round(row["lamisun"]["prefill_tok_s"] / row["dense"]["prefill_tok_s"], 3)
            row["decode_ratio"] = round(row["lamisun"]["decode_tok_s"] / row["dense"]["decode_tok_s"], 3)
        rows.append(row)
    return dict(metric="lamisun_vs_dense_tokens_per_sec", unit="tokens/s", dtype="bf16", data="synthetic",
                sizes=rows)
