"""Prefill and decode throughput of the Fizelix design beside the closest uniform family (Llama: sequential pre-norm
blocks, RMS norm, rotary grouped-query attention, SiLU-gated feed-forward) at equal size, random weights, through the
serving engine (scheduler, paged cache, state slots, decode graphs, sampler). Run as ``python bench.py --fizelix
[SIZE,...]``.

Fizelix: four layers - attention + dense feed-forward, state space + experts, attention + experts, attention + dense -
of which the middle two run twice (six layer runs), a token input of 32 numbers per layer. "Equal size": same width
and vocabulary, as many layers as Fizelix has layer RUNS, the attention's heads, key/value heads and head size; the
dense feed-forward is as wide as the rows a Fizelix token touches in an expert layer (top x expert ff + shared ff).
"""
from __future__ import annotations

import torch

from timisun_compare import measure

SIZES = {
    # width; attention heads / key heads / head size / window / pool; state space heads x value size, state, groups;
    # experts / top / expert ff / shared ff; dense ff
    "w1024": dict(width=1024, heads=8, kv=2, dim=128, window=512, pool=16, sheads=32, svdim=64, state=128, groups=1,
                  experts=16, top=2, eff=512, sff=1024, ff=2048, side=32, vocab=32000),
    "w2048": dict(width=2048, heads=16, kv=4, dim=128, window=512, pool=16, sheads=64, svdim=64, state=128, groups=1,
                  experts=32, top=4, eff=768, sff=1024, ff=4096, side=32, vocab=32000),
    "w4096": dict(width=4096, heads=32, kv=8, dim=128, window=1024, pool=16, sheads=128, svdim=64, state=128,
                  groups=1, experts=64, top=4, eff=1536, sff=2048, ff=8192, side=32, vocab=32000),
}
RUNS = 6  # layer runs of the four layers below (layers 1 and 2 twice)


def fizelix_dict(s):
    dense = dict(kind="dense", ff=s["ff"])
    moe = dict(kind="moe", router=dict(experts=s["experts"], top=s["top"]), expert=dict(ff=s["eff"]),
               shared=dict(ff=s["sff"]))
    att = dict(heads=s["heads"], kv_heads=s["kv"], dim=s["dim"], vdim=s["dim"], scale=s["dim"] ** -0.5,
               mask=dict(size=s["window"], pool=s["pool"]), rot=dict(base=10000.0, dims=s["dim"] // 2))
    ssd = dict(heads=s["sheads"], vdim=s["svdim"], state=s["state"], groups=s["groups"], conv=4, norm_groups=1)
    return dict(architecture="Fizelix", vocab=s["vocab"], width=s["width"], norm=dict(eps=1e-6),
                embedding=dict(scale=1.0), logit_scale=1.0, token_side=dict(dim=s["side"]),
                loop=dict(start=1, stop=3, times=2),
                layers=[dict(type="attention", mixer=att, mlp=dense), dict(type="mamba2", mixer=ssd, mlp=moe),
                        dict(type="attention", mixer=att, mlp=moe), dict(type="attention", mixer=att, mlp=dense)])


def build(kind, s, dev):
    from llmss_amd.models.config import ModelConfig, get_preset
    from llmss_amd.models.layered import create_model
    from llmss_amd.models.weights import random_fizelix_weights, random_weights

    if kind == "fizelix":
        cfg = ModelConfig.from_hf_dict(fizelix_dict(s))
        return create_model(cfg, random_fizelix_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))
    cfg = get_preset("llama2-7b", hidden_size=s["width"], num_layers=RUNS, num_heads=s["heads"],
                     num_kv_heads=s["kv"], head_dim=s["dim"],
                     intermediate_size=(s["top"] * s["eff"] + s["sff"]) // 64 * 64, vocab_size=s["vocab"],
                     max_position_embeddings=8192, rotary_dim=s["dim"])
    return create_model(cfg, random_weights(cfg, device=dev, dtype=torch.bfloat16, seed=1))


def run(sizes, batch, prompt_len, gen_len, rounds, progress, kinds=("fizelix", "dense")):
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
        if "fizelix" in row and "dense" in row:
            row["prefill_ratio"] = round(row["fizelix"]["prefill_tok_s"] / row["dense"]["prefill_tok_s"], 3)
            row["decode_ratio"] = round(row["fizelix"]["decode_tok_s"] / row["dense"]["decode_tok_s"], 3)
        rows.append(row)
    return dict(metric="fizelix_vs_dense_tokens_per_sec", unit="tokens/s", dtype="bf16", data="synthetic",
                sizes=rows)
