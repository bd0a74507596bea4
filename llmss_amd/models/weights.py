"""Canonical rank-local weight layout, tensor-parallel sharding and loading.

One layout serves every family (the decoder in ``decoder.py`` is family-agnostic):

* ``qkv_w``  [nh_l*D + 2*nkv_l*D, H]  column-parallel, q|k|v fused at load time
  (reference loads separate q/k/v for GPT-J, ``gptj_modeling.py:84-92``, and for BigCode loads
  the FULL c_attn on every rank then slices, ``gpt_bigcode_modeling.py:122-155`` - quirk Q8).
* ``o_w``    [H, nh_l*D]  row-parallel; its bias lives on rank 0 only (``layers.py:161-173``).
* ``up_w``   [F_l, H] or, for SwiGLU, [2*F_l, H] with gate/up interleaved in 16-row groups so
  the GEMM epilogue emits silu(gate)*up directly.
* ``down_w`` [H, F_l] row-parallel (bias on rank 0).
* ``wte``    full table replicated on every rank (no embedding all-reduce; reference C1).
* ``head_w`` [Vp/tp, H] vocab-parallel with the vocab padded to a multiple of 16*tp (fixes the
  reference's silent loss of ids >= tp*floor(V/tp), quirk Q6); GPT-J's lm_head bias is loaded
  (the reference drops it, quirk Q5). Tied heads (GPT-2, BigCode) share the checkpoint tensor
  (read once per rank; the reference loads wte twice, Q9).

KV heads: sharded when nkv >= tp, otherwise each rank keeps exactly the kv head(s) its query
heads use (MQA: every rank holds the single kv head), generalising the reference's MQA
replication (``gpt_bigcode_modeling.py:150-155``) to GQA.
"""
from __future__ import annotations

import math
import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import torch

from .. import ops
from ..ops import reference as ref
from .config import ModelConfig


@dataclass
class ShardPlan:
    tp: int
    rank: int
    nh_l: int
    kv_start: int
    nkv_l: int
    F_l: int
    vocab_padded: int

    @property
    def v_l(self) -> int:
        return self.vocab_padded // self.tp


# load neox-RoPE checkpoints with q / k head dims interleaved (gptj-form rotation, fusable into the QKV epilogue)
ROPE_INTERLEAVE = True

def shard_plan(cfg: ModelConfig, tp: int, rank: int) -> ShardPlan:
    nh, nkv = cfg.num_heads, cfg.num_kv_heads
    if nh % tp:
        raise ValueError(f"{cfg.model_type}: num_heads={nh} is not divisible by tp={tp}")
    nh_l = nh // tp
    G = nh // nkv
    kv_start = (rank * nh_l) // G
    kv_end = ((rank + 1) * nh_l - 1) // G + 1
    nkv_l = kv_end - kv_start
    if nh_l % nkv_l or (nh_l // nkv_l) != min(G, nh_l):
        raise ValueError(f"cannot shard {nh} q heads / {nkv} kv heads over tp={tp}")
    if cfg.intermediate_size % tp:
        raise ValueError(f"intermediate_size {cfg.intermediate_size} not divisible by tp={tp}")
    F_l = cfg.intermediate_size // tp
    if cfg.gated_mlp and F_l % 16:
        raise ValueError("gated MLP width per rank must be a multiple of 16")
    vp = math.ceil(cfg.vocab_size / (16 * tp)) * 16 * tp
    return ShardPlan(tp, rank, nh_l, kv_start, nkv_l, F_l, vp)


@dataclass
class Linear:
    # [N, K] bf16, or uint8 fp8-e4m3 when w_scale is set (per-row scales)
    w: torch.Tensor
    b: Optional[torch.Tensor] = None
    w_scale: Optional[torch.Tensor] = None
    glu: bool = False

    def __call__(self, x, act="none", partial_ok=False):
        return ops.linear(x, self.w, self.b, act, self.glu, self.w_scale, partial_ok=partial_ok)

    @property
    def N(self) -> int:
        return self.w.shape[0]

    @property
    def K(self) -> int:
        return self.w.shape[1]

    def rows(self, r0: int, r1: int) -> "Linear":
        """Output features [r0, r1) as a Linear over views (no copy): the weight slice a column chunk of a
        row-parallel projection reads (DecoderLM._reduce_cols)."""
        if self.glu:
            raise ValueError("row slices of SwiGLU linears are not supported")
        return Linear(self.w[r0:r1], None if self.b is None else self.b[r0:r1],
                      None if self.w_scale is None else self.w_scale[r0:r1], False)

    def dense(self) -> torch.Tensor:
        """The [N, K] row-major weight."""
        return self.w

    @property
    def out_features(self):
        return self.N // (2 if self.glu else 1)


@dataclass
class LayerWeights:
    ln1_w: torch.Tensor
    ln1_b: Optional[torch.Tensor]
    ln2_w: Optional[torch.Tensor]
    ln2_b: Optional[torch.Tensor]
    qkv: Linear
    o: Linear
    up: Linear
    down: Linear


@dataclass
class ModelWeights:
    wte: torch.Tensor
    wpe: Optional[torch.Tensor]
    layers: List[LayerWeights]
    lnf_w: torch.Tensor
    lnf_b: Optional[torch.Tensor]
    head: Linear
    cos: Optional[torch.Tensor] = None
    sin: Optional[torch.Tensor] = None
    extra: dict = field(default_factory=dict)
    # neox RoPE models: q / k head dims were interleaved at load (ref.rope_interleave_rows), so the
    # model applies gptj-style RoPE to them (DecoderLM.rope_style)
    rope_interleaved: bool = False

    def nbytes(self) -> int:
        """Device bytes held (views sharing one allocation, like a tied embedding / head, count once)."""
        seen, tot = set(), 0
        for t in _tensors(self):
            st = t.untyped_storage()
            if st.data_ptr() not in seen:
                seen.add(st.data_ptr())
                tot += st.nbytes()
        return tot


def _tensors(mw: ModelWeights):
    yield mw.wte
    if mw.wpe is not None:
        yield mw.wpe
    for L in mw.layers:
        if hasattr(L, "tensors"):  # per-layer designs describe themselves
            yield from L.tensors()
            continue
        for t in (L.ln1_w, L.ln1_b, L.ln2_w, L.ln2_b):
            if t is not None:
                yield t
        for lin in (L.qkv, L.o, L.up, L.down):
            yield lin.w
            if lin.b is not None:
                yield lin.b
    yield mw.lnf_w
    yield mw.head.w
    for t in mw.extra.values():
        if isinstance(t, torch.Tensor):
            yield t


# ------------------------------------------------------------------------------ finalisation
def _finish(cfg: ModelConfig, plan: ShardPlan, wte, wpe, layers_raw, lnf_w, lnf_b, head_w, head_b, device, dtype,
            fp8: bool) -> ModelWeights:
    """Move to device / dtype, pad the head vocab, interleave SwiGLU, optional fp8 quant."""

    def dev(t):
        if t is None:
            return None
        return t.to(device=device, dtype=dtype if t.is_floating_point() else t.dtype).contiguous()

    def lin(w, b, glu=False, quant=False):
        w = dev(w)
        b = dev(b)
        if quant and fp8:
            q, s = ops.quant_fp8_rows(w)
            return Linear(q, b, s, glu)
        return Linear(w, b, None, glu)

    # neox RoPE: interleave the q / k head dims (ROPE_INTERLEAVE = False keeps the checkpoint order; tests)
    il = cfg.position == "rope" and cfg.rope_style == "neox" and ROPE_INTERLEAVE
    layers = []
    for d in layers_raw:
        if il:
            d = dict(d)
            d["qkv_w"] = ref.rope_interleave_rows(d["qkv_w"], plan.nh_l, plan.nkv_l, cfg.head_dim, cfg.rotary_dim)
            if d.get("qkv_b") is not None:
                d["qkv_b"] = ref.rope_interleave_rows(d["qkv_b"], plan.nh_l, plan.nkv_l, cfg.head_dim,
                                                      cfg.rotary_dim)
        if cfg.gated_mlp:
            up_w = ref.glu_interleave(d["gate_w"], d["up_w"], 0)
            up_b = ref.glu_interleave(d["gate_b"], d["up_b"], 0) if d.get("gate_b") is not None else None
        else:
            up_w, up_b = d["up_w"], d.get("up_b")
        layers.append(LayerWeights(
            ln1_w=dev(d["ln1_w"]), ln1_b=dev(d.get("ln1_b")), ln2_w=dev(d.get("ln2_w")), ln2_b=dev(d.get("ln2_b")),
            qkv=lin(d["qkv_w"], d.get("qkv_b"), quant=True), o=lin(d["o_w"], d.get("o_b"), quant=True),
            up=lin(up_w, up_b, glu=cfg.gated_mlp, quant=True), down=lin(d["down_w"], d.get("down_b"), quant=True),
        ))
    # vocab-parallel head with padding
    vl = plan.v_l
    lo = plan.rank * vl
    n = max(0, min(cfg.vocab_size, lo + vl) - lo)
    hb = None
    if head_b is not None:
        hb = torch.zeros(vl, dtype=head_b.dtype, device=head_b.device)
        if n:
            hb[:n] = head_b[lo:lo + n]
    if head_w is wte:
        # tied embedding / head (GPT-2, BigCode): ONE device table [Vpadded, H]; the embedding is its
        # first V rows and this rank's head shard is rows [lo, lo + vl) of it - no second copy in HBM
        # (the reference loads the tied table twice, gpt_bigcode_modeling.py:564,793-797)
        table = torch.zeros(plan.vocab_padded, cfg.hidden_size, dtype=dtype, device=device)
        table[:cfg.vocab_size].copy_(wte.to(device=device, dtype=dtype))
        wte_d, head = table[:cfg.vocab_size], Linear(table[lo:lo + vl], dev(hb))
    else:
        hw = torch.zeros(vl, cfg.hidden_size, dtype=head_w.dtype, device=head_w.device)
        if n:
            hw[:n] = head_w[lo:lo + n]
        wte_d, head = dev(wte), lin(hw, hb)
    mw = ModelWeights(wte=wte_d, wpe=dev(wpe), layers=layers, lnf_w=dev(lnf_w), lnf_b=dev(lnf_b), head=head,
                      rope_interleaved=il)
    if cfg.position == "rope":
        cos, sin = ref.rope_tables(cfg.max_position_embeddings, cfg.rotary_dim, cfg.rope_theta, device)
        mw.cos, mw.sin = cos, sin
    return mw


# ------------------------------------------------------------------------------ random init
def random_weights(cfg: ModelConfig, tp: int = 1, rank: int = 0, device="cpu", dtype=torch.bfloat16,
                   seed: int = 0, std: float = 0.02, fp8: bool = False) -> ModelWeights:
    """Random-init rank-local weights of the architecture (synthetic benches/tests).

    Tensors are generated directly at their rank-local shapes on ``device`` (no full-model
    materialisation). Norm weights are 1, biases small.
    """
    plan = shard_plan(cfg, tp, rank)
    H, D = cfg.hidden_size, cfg.head_dim
    gen_dev = torch.device(device)
    g = torch.Generator(device=gen_dev)
    g.manual_seed(seed * 1000 + rank)
    # replicated tensors (embeddings, norm biases, rank-0 row-parallel biases, the final norm) come
    # from a rank-independent stream: every rank must hold the same copy, as after a checkpoint load
    g_rep = torch.Generator(device=gen_dev)
    g_rep.manual_seed(seed * 1000 + 999)

    def rn(*shape, s=std, rep=False):
        return (torch.randn(*shape, generator=g_rep if rep else g, device=gen_dev, dtype=torch.float32) * s).to(dtype)

    def ones(n):
        return torch.ones(n, device=gen_dev, dtype=dtype)

    layers = []
    qkv_n = (plan.nh_l + 2 * plan.nkv_l) * D
    for _ in range(cfg.num_layers):
        d = dict(
            ln1_w=ones(H), ln1_b=rn(H, rep=True) if cfg.norm == "layernorm" else None,
            qkv_w=rn(qkv_n, H), qkv_b=rn(qkv_n) if cfg.qkv_bias else None,
            o_w=rn(H, plan.nh_l * D, s=std / math.sqrt(2 * cfg.num_layers)),
            o_b=rn(H, rep=True) if cfg.out_bias else None,
            down_w=rn(H, plan.F_l, s=std / math.sqrt(2 * cfg.num_layers)),
            down_b=rn(H, rep=True) if cfg.mlp_bias else None,
        )
        if rank != 0:  # drawn on every rank (keeps the replicated stream aligned), kept on rank 0 only
            d["o_b"] = d["down_b"] = None
        if not cfg.parallel_block:
            d["ln2_w"], d["ln2_b"] = ones(H), (rn(H, rep=True) if cfg.norm == "layernorm" else None)
        if cfg.gated_mlp:
            d["gate_w"], d["up_w"] = rn(plan.F_l, H), rn(plan.F_l, H)
            if cfg.mlp_bias:
                d["gate_b"], d["up_b"] = rn(plan.F_l), rn(plan.F_l)
        else:
            d["up_w"] = rn(plan.F_l, H)
            d["up_b"] = rn(plan.F_l) if cfg.mlp_bias else None
        layers.append(d)
    wte = rn(cfg.vocab_size, H, rep=True)
    wpe = rn(cfg.max_position_embeddings, H, s=0.01, rep=True) if cfg.position == "learned" else None
    if cfg.tie_word_embeddings:
        head_w_full = wte
    else:
        head_w_full = None
    # head shard generated directly (untied) to avoid a full [V, H] second table
    vl = plan.v_l
    lo = rank * vl
    n = max(0, min(cfg.vocab_size, lo + vl) - lo)
    if head_w_full is None:
        head_w = torch.zeros(plan.vocab_padded, H, dtype=dtype, device=gen_dev)
        if n:
            head_w[lo:lo + n] = rn(n, H)
    else:
        head_w = head_w_full
    head_b = None
    if cfg.lm_head_bias:
        head_b = torch.zeros(plan.vocab_padded, dtype=dtype, device=gen_dev)
        if n:
            head_b[lo:lo + n] = rn(n)
    lnf_b = rn(H, rep=True) if cfg.norm == "layernorm" else None
    return _finish(cfg, plan, wte, wpe, layers, ones(H), lnf_b, head_w, head_b, device, dtype, fp8)


# ------------------------------------------------------------------------------ HF checkpoints
def _prefix(reader, *cands):
    for c in cands:
        if any(k.startswith(c) for k in reader.keys()):
            return c
    return ""


def load_hf_weights(cfg: ModelConfig, reader, tp: int = 1, rank: int = 0, device="cpu",
                    dtype=torch.bfloat16, fp8: bool = False) -> ModelWeights:
    """Read a HF checkpoint's tensors for this rank only (sharded reads) and finalise."""
    plan = shard_plan(cfg, tp, rank)
    H, D = cfg.hidden_size, cfg.head_dim
    nh_l, nkv_l = plan.nh_l, plan.nkv_l
    q0, q1 = rank * nh_l * D, (rank + 1) * nh_l * D
    k0, k1 = plan.kv_start * D, (plan.kv_start + nkv_l) * D
    f0, f1 = rank * plan.F_l, (rank + 1) * plan.F_l
    fdt = torch.float32  # read in checkpoint precision, cast once on device
    mt = cfg.model_type
    layers = []

    if mt == "gpt2":
        p = _prefix(reader, "transformer.h.", "h.")
        p = p[:-2] if p else ""
        top = "transformer." if p.startswith("transformer") else ""
        for i in range(cfg.num_layers):
            b = f"{p}h.{i}."
            ca = b + "attn.c_attn."  # Conv1D [H, 3H]
            qkv_w = torch.cat([reader.cols(ca + "weight", q0, q1, fdt), reader.cols(ca + "weight", H + k0, H + k1, fdt),
                               reader.cols(ca + "weight", 2 * H + k0, 2 * H + k1, fdt)], 1).t()
            cb = reader.get(ca + "bias", fdt)
            qkv_b = torch.cat([cb[q0:q1], cb[H + k0:H + k1], cb[2 * H + k0:2 * H + k1]])
            layers.append(dict(
                ln1_w=reader.get(b + "ln_1.weight"), ln1_b=reader.get(b + "ln_1.bias"),
                ln2_w=reader.get(b + "ln_2.weight"), ln2_b=reader.get(b + "ln_2.bias"),
                qkv_w=qkv_w, qkv_b=qkv_b,
                o_w=reader.rows(b + "attn.c_proj.weight", q0, q1, fdt).t(),
                o_b=reader.get(b + "attn.c_proj.bias") if rank == 0 else None,
                up_w=reader.cols(b + "mlp.c_fc.weight", f0, f1, fdt).t(),
                up_b=reader.get(b + "mlp.c_fc.bias", fdt)[f0:f1],
                down_w=reader.rows(b + "mlp.c_proj.weight", f0, f1, fdt).t(),
                down_b=reader.get(b + "mlp.c_proj.bias") if rank == 0 else None,
            ))
        wte = reader.get(top + "wte.weight")
        wpe = reader.get(top + "wpe.weight")
        lnf_w, lnf_b = reader.get(top + "ln_f.weight"), reader.get(top + "ln_f.bias")
        head_w = reader.get("lm_head.weight") if (not cfg.tie_word_embeddings and reader.has("lm_head.weight")) else wte
        head_b = None
    elif mt == "gptj":
        for i in range(cfg.num_layers):
            b = f"transformer.h.{i}."
            a = b + "attn."
            qkv_w = torch.cat([reader.rows(a + "q_proj.weight", q0, q1, fdt), reader.rows(a + "k_proj.weight", k0, k1, fdt),
                               reader.rows(a + "v_proj.weight", k0, k1, fdt)], 0)
            layers.append(dict(
                ln1_w=reader.get(b + "ln_1.weight"), ln1_b=reader.get(b + "ln_1.bias"),
                qkv_w=qkv_w, o_w=reader.cols(a + "out_proj.weight", q0, q1, fdt),
                up_w=reader.rows(b + "mlp.fc_in.weight", f0, f1, fdt), up_b=reader.get(b + "mlp.fc_in.bias")[f0:f1],
                down_w=reader.cols(b + "mlp.fc_out.weight", f0, f1, fdt),
                down_b=reader.get(b + "mlp.fc_out.bias") if rank == 0 else None,
            ))
        wte = reader.get("transformer.wte.weight")
        wpe = None
        lnf_w, lnf_b = reader.get("transformer.ln_f.weight"), reader.get("transformer.ln_f.bias")
        head_w = reader.get("lm_head.weight")
        head_b = reader.get("lm_head.bias") if reader.has("lm_head.bias") else None
    elif mt == "gpt_bigcode":
        nkv = cfg.num_kv_heads
        for i in range(cfg.num_layers):
            b = f"transformer.h.{i}."
            ca = b + "attn.c_attn."
            if nkv == cfg.num_heads:
                # MHA: nn.Linear [3H, H] laid out per head as [q_h | k_h | v_h] (HF view(nh, 3D))
                h0, h1 = rank * nh_l, (rank + 1) * nh_l
                blk = reader.rows(ca + "weight", 3 * D * h0, 3 * D * h1, fdt).view(nh_l, 3, D, H)
                qkv_w = torch.cat([blk[:, 0].reshape(-1, H), blk[:, 1].reshape(-1, H), blk[:, 2].reshape(-1, H)], 0)
                bb = reader.get(ca + "bias", fdt)[3 * D * h0:3 * D * h1].view(nh_l, 3, D)
                qkv_b = torch.cat([bb[:, 0].reshape(-1), bb[:, 1].reshape(-1), bb[:, 2].reshape(-1)])
            else:
                # MQA/GQA: nn.Linear [H + 2*nkv*D, H] = [q | k | v]
                kb, vb = H, H + nkv * D
                qkv_w = torch.cat([reader.rows(ca + "weight", q0, q1, fdt),
                                   reader.rows(ca + "weight", kb + k0, kb + k1, fdt),
                                   reader.rows(ca + "weight", vb + k0, vb + k1, fdt)], 0)
                cb = reader.get(ca + "bias", fdt)
                qkv_b = torch.cat([cb[q0:q1], cb[kb + k0:kb + k1], cb[vb + k0:vb + k1]])
            layers.append(dict(
                ln1_w=reader.get(b + "ln_1.weight"), ln1_b=reader.get(b + "ln_1.bias"),
                ln2_w=reader.get(b + "ln_2.weight"), ln2_b=reader.get(b + "ln_2.bias"),
                qkv_w=qkv_w, qkv_b=qkv_b,
                o_w=reader.cols(b + "attn.c_proj.weight", q0, q1, fdt),
                o_b=reader.get(b + "attn.c_proj.bias") if rank == 0 else None,
                up_w=reader.rows(b + "mlp.c_fc.weight", f0, f1, fdt), up_b=reader.get(b + "mlp.c_fc.bias")[f0:f1],
                down_w=reader.cols(b + "mlp.c_proj.weight", f0, f1, fdt),
                down_b=reader.get(b + "mlp.c_proj.bias") if rank == 0 else None,
            ))
        wte = reader.get("transformer.wte.weight")
        wpe = reader.get("transformer.wpe.weight")
        lnf_w, lnf_b = reader.get("transformer.ln_f.weight"), reader.get("transformer.ln_f.bias")
        head_w = reader.get("lm_head.weight") if (not cfg.tie_word_embeddings and reader.has("lm_head.weight")) else wte
        head_b = None
    elif mt == "llama":
        for i in range(cfg.num_layers):
            b = f"model.layers.{i}."
            a = b + "self_attn."
            d = dict(
                ln1_w=reader.get(b + "input_layernorm.weight"), ln2_w=reader.get(b + "post_attention_layernorm.weight"),
                qkv_w=torch.cat([reader.rows(a + "q_proj.weight", q0, q1, fdt), reader.rows(a + "k_proj.weight", k0, k1, fdt),
                                 reader.rows(a + "v_proj.weight", k0, k1, fdt)], 0),
                o_w=reader.cols(a + "o_proj.weight", q0, q1, fdt),
                gate_w=reader.rows(b + "mlp.gate_proj.weight", f0, f1, fdt),
                up_w=reader.rows(b + "mlp.up_proj.weight", f0, f1, fdt),
                down_w=reader.cols(b + "mlp.down_proj.weight", f0, f1, fdt),
            )
            if cfg.qkv_bias:
                d["qkv_b"] = torch.cat([reader.get(a + "q_proj.bias")[q0:q1], reader.get(a + "k_proj.bias")[k0:k1],
                                        reader.get(a + "v_proj.bias")[k0:k1]])
            if cfg.out_bias and rank == 0:
                d["o_b"] = reader.get(a + "o_proj.bias")
            layers.append(d)
        wte = reader.get("model.embed_tokens.weight")
        wpe = None
        lnf_w, lnf_b = reader.get("model.norm.weight"), None
        head_w = wte if cfg.tie_word_embeddings or not reader.has("lm_head.weight") else reader.get("lm_head.weight")
        head_b = None
    else:
        raise ValueError(mt)
    return _finish(cfg, plan, wte, wpe, layers, lnf_w, lnf_b, head_w, head_b, device, dtype, fp8)


# ------------------------------------------------------------------------------ per-rank shard cache
# a restart of a large TP deployment should not re-read, re-shard, re-interleave and
# re-quantize the HF checkpoint on every rank. The finished per-rank weights (this rank's shards,
# padded head, SwiGLU interleave, fp8 + scales) are written once as one safetensors file per rank
# and mmap-loaded by the native reader afterwards.
def _flat(mw: ModelWeights) -> Dict[str, torch.Tensor]:
    out: Dict[str, torch.Tensor] = {"wte": mw.wte, "lnf_w": mw.lnf_w}
    if mw.wpe is not None:
        out["wpe"] = mw.wpe
    if mw.lnf_b is not None:
        out["lnf_b"] = mw.lnf_b

    def put_lin(pfx, lin: Linear):
        out[pfx + ".w"] = lin.dense().contiguous()  # shards are stored row-major
        if lin.b is not None:
            out[pfx + ".b"] = lin.b
        if lin.w_scale is not None:
            out[pfx + ".s"] = lin.w_scale

    for i, L in enumerate(mw.layers):
        for nm in ("ln1_w", "ln1_b", "ln2_w", "ln2_b"):
            t = getattr(L, nm)
            if t is not None:
                out[f"l{i}.{nm}"] = t
        for nm in ("qkv", "o", "up", "down"):
            put_lin(f"l{i}.{nm}", getattr(L, nm))
    put_lin("head", mw.head)
    return out


def save_shard(mw: ModelWeights, path: str) -> None:
    from safetensors.torch import save_file

    # clone: a tied head is a view of the embedding table (safetensors refuses shared storage)
    tensors = {k: v.detach().cpu().contiguous().clone() for k, v in _flat(mw).items()}
    meta = {"format": "llmss_amd-shard-v1", "layers": str(len(mw.layers)),
            "glu": str(int(mw.layers[0].up.glu)) if mw.layers else "0",
            "rope_interleaved": str(int(mw.rope_interleaved))}
    if mw.head.w.untyped_storage().data_ptr() == mw.wte.untyped_storage().data_ptr():
        es = mw.wte.element_size()
        meta["tied_head_row"] = str((mw.head.w.data_ptr() - mw.wte.data_ptr()) // (es * mw.wte.shape[1]))
        meta["tied_table_rows"] = str(mw.wte.untyped_storage().nbytes() // (es * mw.wte.shape[1]))
    os.makedirs(os.path.dirname(path) or ".", exist_ok=True)
    tmp = path + f".tmp{os.getpid()}"
    save_file(tensors, tmp, metadata=meta)
    os.replace(tmp, path)  # atomic: a concurrent reader never sees a partial file


def load_shard(cfg: ModelConfig, path: str, device, dtype) -> ModelWeights:
    from ..utils.checkpoint import CheckpointReader

    rd = CheckpointReader([path])
    names = set(rd.routing)

    def get(name):
        if name not in names:
            return None
        t = rd.get(name)
        return t.to(device=device, dtype=dtype if t.is_floating_point() and t.dtype != torch.float32 else t.dtype)

    def lin(pfx, glu=False):
        s = rd.get(pfx + ".s").to(device) if pfx + ".s" in names else None
        w = rd.get(pfx + ".w").to(device)
        if s is None and w.is_floating_point():
            w = w.to(dtype)
        return Linear(w, get(pfx + ".b"), s, glu)

    layers = []
    for i in range(cfg.num_layers):
        layers.append(LayerWeights(get(f"l{i}.ln1_w"), get(f"l{i}.ln1_b"), get(f"l{i}.ln2_w"), get(f"l{i}.ln2_b"),
                                   lin(f"l{i}.qkv"), lin(f"l{i}.o"), lin(f"l{i}.up", glu=cfg.gated_mlp),
                                   lin(f"l{i}.down")))
    head, wte = lin("head"), get("wte")
    meta = rd.metadata()
    if "tied_head_row" in meta:  # re-tie: one [Vpadded, H] table, embedding and head shard are views of it
        lo, rows = int(meta["tied_head_row"]), int(meta["tied_table_rows"])
        table = torch.zeros(rows, wte.shape[1], dtype=wte.dtype, device=wte.device)
        table[:wte.shape[0]] = wte
        wte, head = table[:wte.shape[0]], Linear(table[lo:lo + head.w.shape[0]], head.b, head.w_scale, head.glu)
    mw = ModelWeights(wte=wte, wpe=get("wpe"), layers=layers, lnf_w=get("lnf_w"), lnf_b=get("lnf_b"), head=head,
                      rope_interleaved=meta.get("rope_interleaved", "0") == "1")
    if cfg.position == "rope":
        mw.cos, mw.sin = ref.rope_tables(cfg.max_position_embeddings, cfg.rotary_dim, cfg.rope_theta, device)
    return mw


def shard_cache_path(root: str, model_dir: str, files: List[str], tp: int, rank: int, dtype: torch.dtype,
                     fp8: bool) -> str:
    """Cache file for (checkpoint identity, TP layout, dtype); identity = paths + sizes + mtimes."""
    import hashlib

    h = hashlib.sha1(os.path.abspath(model_dir).encode())
    for f in sorted(files):
        st = os.stat(f)
        h.update(f"{os.path.basename(f)}:{st.st_size}:{int(st.st_mtime)}".encode())
    tag = str(dtype).replace("torch.", "") + ("-fp8" if fp8 else "")
    return os.path.join(root, h.hexdigest()[:16], f"tp{tp}-r{rank}-{tag}.safetensors")


# ------------------------------------------------------------------------------ per-layer designs (Timisun)
@dataclass
class LatentAttnWeights:
    """Latent attention: ``qc`` [heads * dim (+ kv_rank), H] is the query projection followed, in a layer that
    projects its own latent rows (``own_kv``), by the latent down-projection - one GEMM for both; ``kv_norm``
    [kv_rank] the latent's plain RMS-norm weight; ``uk_t`` [heads, kv_rank, dim] the key up-projection, per head
    transposed (the absorbed query is q_h . uk_h: dim is then the contiguous contraction index); ``uv``
    [heads * vdim, kv_rank] the value up-projection; ``o`` [H, heads * vdim]."""
    qc: torch.Tensor
    own_kv: bool
    kv_norm: Optional[torch.Tensor]
    uk_t: torch.Tensor
    uv: torch.Tensor
    o: torch.Tensor
    # with a rotated part: every query head holds dim + rot_dim rows in ``qc``, the down-projection rot_dim more rows
    # after the latent's; ``freqs`` fp32 [rot_dim / 2] are the pairs' angular steps per position. ``gate_col``: first
    # row of the output gate's projection inside ``qc`` (None: no gate). Rows of ``qc`` are padded to a multiple of 8.
    freqs: Optional[torch.Tensor] = None
    gate_col: Optional[int] = None
    rot_key: Optional[tuple] = None  # (dims, base): layers with the same rotation share a step's angles

    def tensors(self):
        return [t for t in (self.qc, self.kv_norm, self.uk_t, self.uv, self.o, self.freqs) if t is not None]


@dataclass
class MoEWeights:
    """Experts stacked: ``gate`` / ``up`` [E, F, H], ``down`` [E, H, F]; ``router`` [E, H]; ``correction`` fp32 [E]
    (added to the scores for the choice only); the shared expert as one gate | up matrix ``shared_gu`` [2 Fs, H]
    and ``shared_down`` [H, Fs]."""
    router: torch.Tensor
    correction: Optional[torch.Tensor]
    gate: torch.Tensor
    up: torch.Tensor
    down: torch.Tensor
    shared_gu: Optional[torch.Tensor] = None
    shared_down: Optional[torch.Tensor] = None

    def tensors(self):
        return [t for t in (self.router, self.correction, self.gate, self.up, self.down, self.shared_gu,
                            self.shared_down) if t is not None]


@dataclass
class BlockWeights:
    """One parallel block of a per-layer design: a single norm feeding the mixer and the feed-forward."""
    norm1: torch.Tensor
    mix: LatentAttnWeights
    mlp: Optional[MoEWeights]

    def tensors(self):
        return [self.norm1] + self.mix.tensors() + (self.mlp.tensors() if self.mlp else [])


def _tied_head(cfg: ModelConfig, wte: torch.Tensor, device, dtype):
    """One device table [V padded to 16, H]: the embedding is its first V rows, the head the whole of it."""
    vp = math.ceil(cfg.vocab_size / 16) * 16
    table = torch.zeros(vp, cfg.hidden_size, dtype=dtype, device=device)
    table[:cfg.vocab_size].copy_(wte.to(device=device, dtype=dtype))
    return table[:cfg.vocab_size], Linear(table)


def _heads_t(uk: torch.Tensor, heads: int, dim: int, rank: int, layer: int) -> torch.Tensor:
    if tuple(uk.shape) != (heads * dim, rank):
        raise ValueError(f"layer {layer}: uk has shape {tuple(uk.shape)}, the config says {(heads * dim, rank)}")
    return uk.view(heads, dim, rank).transpose(1, 2).contiguous()


def _timisun_finish(cfg: ModelConfig, get, device, dtype) -> ModelWeights:
    """``get(name)`` returns the checkpoint tensor of that name (CPU); tensor names as in the checkpoint:
    ``embed``, ``final.norm``, ``l<i>.norm1``, ``l<i>.mix.{q,dkv,dkv.norm,uk,uv,o}``,
    ``l<i>.mlp.{router,correction,e<k>.{gate,up,down},shared.{gate,up,down}}``."""
    def dev(t, dt=dtype):
        return t.to(device=device, dtype=dt).contiguous()

    layers = []
    for i, spec in enumerate(cfg.layer_specs):
        p = f"l{i}."
        mx = spec.mixer
        own = mx.kv_from is None
        q = get(p + "mix.q")
        mix = LatentAttnWeights(
            qc=dev(torch.cat([q, get(p + "mix.dkv")], 0) if own else q), own_kv=own,
            kv_norm=dev(get(p + "mix.dkv.norm")) if own else None,
            uk_t=dev(_heads_t(get(p + "mix.uk"), mx.heads, mx.dim, mx.kv_rank, i)), uv=dev(get(p + "mix.uv")),
            o=dev(get(p + "mix.o")))
        want = {"qc": (mx.heads * mx.dim + (mx.kv_rank if own else 0), cfg.hidden_size),
                "uk_t": (mx.heads, mx.kv_rank, mx.dim), "uv": (mx.heads * mx.vdim, mx.kv_rank),
                "o": (cfg.hidden_size, mx.heads * mx.vdim)}
        for nm, shp in want.items():
            if tuple(getattr(mix, nm).shape) != shp:
                raise ValueError(f"layer {i}: {nm} has shape {tuple(getattr(mix, nm).shape)}, the config says {shp}")
        mlp = None
        if spec.mlp is not None:
            f, m = spec.mlp, p + "mlp."
            E = f.experts
            sh_gu = sh_down = None
            if f.shared is not None:
                sh_gu = dev(torch.cat([get(m + "shared.gate"), get(m + "shared.up")], 0))
                sh_down = dev(get(m + "shared.down"))
            mlp = MoEWeights(
                router=dev(get(m + "router")), correction=dev(get(m + "correction"), torch.float32),
                gate=dev(torch.stack([get(f"{m}e{k}.gate") for k in range(E)])),
                up=dev(torch.stack([get(f"{m}e{k}.up") for k in range(E)])),
                down=dev(torch.stack([get(f"{m}e{k}.down") for k in range(E)])),
                shared_gu=sh_gu, shared_down=sh_down)
            if tuple(mlp.gate.shape) != (E, f.expert.ff, cfg.hidden_size):
                raise ValueError(f"layer {i}: expert gate {tuple(mlp.gate.shape)} does not fit the config")
        layers.append(BlockWeights(dev(get(p + "norm1")), mix, mlp))
    wte, head = _tied_head(cfg, get("embed"), device, dtype)
    return ModelWeights(wte=wte, wpe=None, layers=layers, lnf_w=dev(get("final.norm")), lnf_b=None, head=head)


def load_timisun_weights(cfg: ModelConfig, reader, device="cpu", dtype=torch.bfloat16) -> ModelWeights:
    return _timisun_finish(cfg, lambda n: reader.get(n), device, dtype)


def random_timisun_weights(cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, seed: int = 0) -> ModelWeights:
    """Random-init weights of a per-layer (Timisun) config: projections ~ N(0, 1 / fan_in), norm weights and the
    router's correction small around zero, values rounded to bf16 (so a bf16 and an fp32 run hold the same model)."""
    gen = device if torch.device(device).type == "cuda" else "cpu"  # large models: draw on the GPU
    return _timisun_finish(cfg, _timisun_random(cfg, seed, gen), device, dtype)


def timisun_state_dict(cfg: ModelConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """The random weights of :func:`random_timisun_weights` under their checkpoint names (bf16; tests, examples)."""
    get = _timisun_random(cfg, seed)
    names = ["embed", "final.norm"]
    for i, spec in enumerate(cfg.layer_specs):
        p = f"l{i}."
        names += [p + "norm1", p + "mix.q", p + "mix.uk", p + "mix.uv", p + "mix.o"]
        if spec.mixer.kv_from is None:
            names += [p + "mix.dkv", p + "mix.dkv.norm"]
        if spec.mlp is not None:
            names += [p + "mlp.router", p + "mlp.correction"]
            for k in range(spec.mlp.experts):
                names += [f"{p}mlp.e{k}.{n}" for n in ("gate", "up", "down")]
            if spec.mlp.shared is not None:
                names += [f"{p}mlp.shared.{n}" for n in ("gate", "up", "down")]
    return {n: get(n).to(torch.bfloat16) for n in names}


def _timisun_random(cfg: ModelConfig, seed: int, device="cpu"):
    import zlib

    W = cfg.hidden_size

    def shape_of(name: str):
        if name == "embed":
            return (cfg.vocab_size, W), 1.0 / cfg.embedding_scale
        if name == "final.norm":
            return (W,), 0.1
        i = int(name[1:name.index(".")])
        spec, rest = cfg.layer_specs[i], name[name.index(".") + 1:]
        mx, f = spec.mixer, spec.mlp
        if rest == "norm1":
            return (W,), 0.1
        if rest == "mix.q":
            return (mx.heads * mx.dim, W), W ** -0.5
        if rest == "mix.dkv":
            return (mx.kv_rank, W), W ** -0.5
        if rest == "mix.dkv.norm":
            return (mx.kv_rank,), None  # around one
        if rest == "mix.uk":
            return (mx.heads * mx.dim, mx.kv_rank), mx.kv_rank ** -0.5 / max(mx.scale, 1e-6) / mx.dim ** 0.5
        if rest == "mix.uv":
            return (mx.heads * mx.vdim, mx.kv_rank), mx.kv_rank ** -0.5
        if rest == "mix.o":
            return (W, mx.heads * mx.vdim), (mx.heads * mx.vdim) ** -0.5
        if rest == "mlp.router":
            return (f.experts, W), W ** -0.5
        if rest == "mlp.correction":
            return (f.experts,), 0.1
        part = rest.split(".")[-1]
        e = f.shared if ".shared." in rest else f.expert
        return ((W, e.ff), e.ff ** -0.5) if part == "down" else ((e.ff, W), W ** -0.5)

    def get(name: str) -> torch.Tensor:
        g = torch.Generator(device=device)
        g.manual_seed((seed * 1000003 + zlib.crc32(name.encode())) & 0x7FFFFFFF)
        shp, std = shape_of(name)
        t = torch.randn(*shp, generator=g, dtype=torch.float32, device=device)
        t = 1.0 + 0.1 * t if std is None else t * std
        return t.to(torch.bfloat16).float()
    return get


# ------------------------------------------------------------------------------ sequential per-layer designs (Babotar)
@dataclass
class StreamWeights:
    """Read / write / mix weights of one sublayer over the residual streams (fp32): u = sum_s inw[s] x_s;
    x_t <- sum_s mix[s, t] x_s + c * outw[t] * y."""
    inw: torch.Tensor
    outw: torch.Tensor
    mix: torch.Tensor

    def tensors(self):
        return [self.inw, self.outw, self.mix]


@dataclass
class ParallelMixWeights:
    """Attention beside a gated delta rule, both reading the same rows. ``proj`` [N padded to 8, W] holds every input
    projection of the two as one matrix (one GEMM); ``cols`` names the first column of each part: lq, lk, lv (the
    attention's q, k, v, contiguous), rq, rk, rv (the delta rule's, contiguous: one convolution runs over them), rg
    (its output gate), rb, ra (its per-head write strength and decay inputs). ``bias`` [lq | lk | lv] or None;
    ``talk`` fp32 [heads, heads] or None; ``angles`` fp32 [positions, rot / 2, 2] or None; ``conv`` [rq | rk | rv
    channels, taps]; ``A_log``, ``dt_bias`` fp32 [heads]; ``norm`` [vdim]; ``o`` [W, left width + right width], the
    two output projections side by side (one GEMM over the concatenated branch outputs)."""
    proj: torch.Tensor
    cols: Dict[str, int]
    bias: Optional[torch.Tensor]
    talk: Optional[torch.Tensor]
    angles: Optional[torch.Tensor]
    conv: torch.Tensor
    A_log: torch.Tensor
    dt_bias: torch.Tensor
    norm: torch.Tensor
    o: torch.Tensor

    def tensors(self):
        return [t for t in (self.proj, self.bias, self.talk, self.angles, self.conv, self.A_log, self.dt_bias, self.norm,
                            self.o) if t is not None]


@dataclass
class DecayMixWeights:
    """Decay linear attention: ``proj`` [q | k | v | g rows padded to 8, W], ``decay`` fp32 [heads], ``norm``
    [heads * vdim], ``o`` [W, heads * vdim]."""
    proj: torch.Tensor
    cols: Dict[str, int]
    decay: torch.Tensor
    norm: torch.Tensor
    o: torch.Tensor

    def tensors(self):
        return [self.proj, self.decay, self.norm, self.o]


@dataclass
class DenseMLPWeights:
    """``gu`` [2 ff, W]: gate rows, then up rows (an ungated feed-forward: [ff, W], the up rows alone); ``down``
    [W, ff]; ``act_params``: the activation's learned numbers in the form the kernel takes (xIELU: softplus(p),
    1/2 + softplus(q))."""
    gu: torch.Tensor
    down: torch.Tensor
    act_params: tuple = ()

    def tensors(self):
        return [self.gu, self.down]


@dataclass
class SeqBlockWeights:
    """One sequential block: norm1 -> (input convolution) -> mixer, norm2 -> feed-forward, each over the streams."""
    norm1: torch.Tensor
    norm2: Optional[torch.Tensor]
    hc1: StreamWeights
    hc2: Optional[StreamWeights]
    canon: Optional[torch.Tensor]
    mix: object
    mlp: Optional[DenseMLPWeights]

    def tensors(self):
        out = [self.norm1] + self.hc1.tensors() + self.mix.tensors()
        for t in (self.norm2, self.canon):
            if t is not None:
                out.append(t)
        if self.hc2 is not None:
            out += self.hc2.tensors()
        if self.mlp is not None:
            out += self.mlp.tensors()
        return out


def babotar_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names of a Babotar config and their shapes."""
    W, S = cfg.hidden_size, cfg.streams
    out = {"embed": (cfg.vocab_size, W), "pos": (cfg.max_position_embeddings, W), "final.norm": (W,),
           "head": (cfg.vocab_size, W)}
    for i, spec in enumerate(cfg.layer_specs):
        p = f"l{i}."
        out[p + "norm1"] = (W,)
        subs = (1, 2) if spec.mlp is not None else (1,)
        if S:
            for q in subs:
                out.update({f"{p}hc{q}.in": (S,), f"{p}hc{q}.out": (S,), f"{p}hc{q}.mix": (S, S)})
        if cfg.canon_taps:
            out[p + "canon1"] = (W, cfg.canon_taps)
        m = spec.mixer
        if m.kind == "lightning":
            out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W),
                        p + "mix.v": (m.heads * m.vdim, W), p + "mix.g": (m.heads * m.vdim, W),
                        p + "mix.o": (W, m.heads * m.vdim), p + "mix.norm": (m.heads * m.vdim,)})
        else:
            a, r, pl, pr = m.left, m.right, p + "mix.left.", p + "mix.right."
            out.update({pl + "q": (a.heads * a.dim, W), pl + "k": (a.kv_heads * a.dim, W),
                        pl + "v": (a.kv_heads * a.vdim, W), pl + "o": (W, a.heads * a.vdim)})
            if a.bias:
                out.update({pl + "q.b": (a.heads * a.dim,), pl + "k.b": (a.kv_heads * a.dim,),
                            pl + "v.b": (a.kv_heads * a.vdim,)})
            if a.talk:
                out[pl + "talk"] = (a.heads, a.heads)
            out.update({pr + "q": (r.kv_heads * r.dim, W), pr + "q.conv": (r.kv_heads * r.dim, r.conv),
                        pr + "k": (r.kv_heads * r.dim, W), pr + "k.conv": (r.kv_heads * r.dim, r.conv),
                        pr + "v": (r.heads * r.vdim, W), pr + "v.conv": (r.heads * r.vdim, r.conv),
                        pr + "b": (r.heads, W), pr + "a": (r.heads, W), pr + "A_log": (r.heads,),
                        pr + "dt_bias": (r.heads,), pr + "norm": (r.vdim,), pr + "g": (r.heads * r.vdim, W),
                        pr + "o": (W, r.heads * r.vdim)})
        if spec.mlp is not None:
            out.update({p + "norm2": (W,), p + "mlp.gate": (spec.mlp.ff, W), p + "mlp.up": (spec.mlp.ff, W),
                        p + "mlp.down": (W, spec.mlp.ff)})
    return out


def _cat_rows(parts, pad_to: int = 8):
    """(matrix of the parts' rows one after the other, zero rows up to a multiple of ``pad_to``; first row of each)."""
    cols, n = {}, 0
    for name, t in parts:
        cols[name] = n
        n += t.shape[0]
    mats = [t for _, t in parts]
    if n % pad_to:
        mats.append(torch.zeros(pad_to - n % pad_to, mats[0].shape[1], dtype=mats[0].dtype))
    return torch.cat(mats, 0), cols


def _babotar_finish(cfg: ModelConfig, get, has, device, dtype) -> ModelWeights:
    """``get(name)`` returns the checkpoint tensor of that name (CPU), ``has(name)`` whether it exists. Shapes are
    checked against the config; the head-mixing matrix and the q / k / v biases are optional tensors."""
    from ..ops.reference import rope_angle_table

    shapes = babotar_shapes(cfg)
    optional = (".talk", ".q.b", ".k.b", ".v.b")

    def g(name):
        t = get(name)
        if tuple(t.shape) != shapes[name]:
            raise ValueError(f"{name} has shape {tuple(t.shape)}, the config says {shapes[name]}")
        return t

    def opt(name):
        return g(name) if has(name) else None

    def dev(t, dt=dtype):
        return None if t is None else t.to(device=device, dtype=dt).contiguous()

    def f32(t):
        return dev(t, torch.float32)
    W, S = cfg.hidden_size, cfg.streams
    one = StreamWeights(f32(torch.ones(1)), f32(torch.ones(1)), f32(torch.ones(1, 1)))
    tables = {}
    layers = []
    for i, spec in enumerate(cfg.layer_specs):
        p = f"l{i}."

        def hc(q):
            return StreamWeights(f32(g(f"{p}hc{q}.in")), f32(g(f"{p}hc{q}.out")), f32(g(f"{p}hc{q}.mix"))) if S else one
        m = spec.mixer
        if m.kind == "lightning":
            proj, cols = _cat_rows([(n, g(p + "mix." + n)) for n in ("q", "k", "v", "g")])
            mix = DecayMixWeights(dev(proj), cols, f32(torch.tensor(m.decay)), dev(g(p + "mix.norm")),
                                  dev(g(p + "mix.o")))
        else:
            a, pl, pr = m.left, p + "mix.left.", p + "mix.right."
            proj, cols = _cat_rows([("lq", g(pl + "q")), ("lk", g(pl + "k")), ("lv", g(pl + "v")),
                                    ("rq", g(pr + "q")), ("rk", g(pr + "k")), ("rv", g(pr + "v")),
                                    ("rg", g(pr + "g")), ("rb", g(pr + "b")), ("ra", g(pr + "a"))])
            bias = None
            if any(has(pl + n + ".b") for n in "qkv"):
                bias = torch.cat([g(pl + n + ".b") if has(pl + n + ".b") else torch.zeros(shapes[pl + n][0])
                                  for n in "qkv"])
            angles = None
            if a.rot is not None and a.rot.dims:
                key = (a.rot.dims, a.rot.base, a.rot.scaling)
                if key not in tables:
                    tables[key] = dev(rope_angle_table(cfg.max_position_embeddings, *key), torch.float32)
                angles = tables[key]
            mix = ParallelMixWeights(
                dev(proj), cols, dev(bias), f32(opt(pl + "talk")), angles,
                dev(torch.cat([g(pr + n + ".conv") for n in "qkv"], 0)), f32(g(pr + "A_log")), f32(g(pr + "dt_bias")),
                dev(g(pr + "norm")), dev(torch.cat([g(pl + "o"), g(pr + "o")], 1)))
        mlp = None
        if spec.mlp is not None:
            mlp = DenseMLPWeights(dev(torch.cat([g(p + "mlp.gate"), g(p + "mlp.up")], 0)), dev(g(p + "mlp.down")))
        layers.append(SeqBlockWeights(
            dev(g(p + "norm1")), dev(g(p + "norm2")) if mlp is not None else None, hc(1),
            hc(2) if mlp is not None else None, dev(g(p + "canon1")) if cfg.canon_taps else None, mix, mlp))
    vp = math.ceil(cfg.vocab_size / 16) * 16
    head = torch.zeros(vp, W, dtype=dtype, device=device)
    head[:cfg.vocab_size].copy_(g("head").to(device=device, dtype=dtype))
    return ModelWeights(wte=dev(g("embed")), wpe=dev(g("pos")) if has("pos") else None, layers=layers,
                        lnf_w=dev(g("final.norm")), lnf_b=None, head=Linear(head))


def load_babotar_weights(cfg: ModelConfig, reader, device="cpu", dtype=torch.bfloat16) -> ModelWeights:
    names = set(reader.keys())
    return _babotar_finish(cfg, lambda n: reader.get(n), lambda n: n in names, device, dtype)


def _babotar_random(cfg: ModelConfig, seed: int, device="cpu"):
    import zlib

    shapes = babotar_shapes(cfg)

    def get(name: str) -> torch.Tensor:
        g = torch.Generator(device=device)
        g.manual_seed((seed * 1000003 + zlib.crc32(name.encode())) & 0x7FFFFFFF)
        shp = shapes[name]
        t = torch.randn(*shp, generator=g, dtype=torch.float32, device=device)
        last = name.split(".")[-1]
        if last.startswith("norm") or name == "final.norm":
            t = 1.0 + 0.1 * t
        elif name == "pos":
            t = 0.3 * t
        elif last in ("in", "out"):
            t = 1.0 / max(1, cfg.streams) + 0.2 * t if last == "in" else 1.0 + 0.2 * t
        elif last == "mix":
            t = torch.eye(shp[0], device=device) + 0.15 * t
        elif last == "talk":
            t = torch.eye(shp[0], device=device) + 0.2 * t
        elif last in ("conv", "canon1"):
            t = t * shp[1] ** -0.5
        elif last == "A_log":
            t = 0.5 * t - 1.0
        elif last in ("dt_bias", "b") and len(shp) == 1:
            t = 0.3 * t
        elif len(shp) == 2 and name not in ("embed",):
            t = t * shp[1] ** -0.5
        return t.to(torch.bfloat16).float()
    return get


def random_babotar_weights(cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, seed: int = 0) -> ModelWeights:
    """Random-init weights of a Babotar config (values rounded to bf16, so a bf16 and an fp32 run hold the same
    model): projections ~ N(0, 1 / fan_in), norm weights around one, stream weights around the plain residual."""
    return _babotar_finish(cfg, _babotar_random(cfg, seed), lambda n: True, device, dtype)


def babotar_state_dict(cfg: ModelConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """The random weights of :func:`random_babotar_weights` under their checkpoint names (bf16; tests, examples)."""
    get = _babotar_random(cfg, seed)
    return {n: get(n).to(torch.bfloat16) for n in babotar_shapes(cfg)}


# ------------------------------------------------------------------------------ post-norm per-layer designs (Lamisun)
@dataclass
class DiffAttnWeights:
    """Differential attention: ``proj`` [q | k | v rows padded to 8, W] (q: heads x 2 maps x dim, k: kv_heads x 2
    maps x dim, v: kv_heads x vdim), ``cols`` the first row of each part; ``q_norm`` / ``k_norm`` [dim] or None;
    ``lam``: the weight of the second map, exp(lq1 . lk1) - exp(lq2 . lk2) + diff, formed once in fp32; ``o``
    [W, heads * vdim]."""
    proj: torch.Tensor
    cols: Dict[str, int]
    q_norm: Optional[torch.Tensor]
    k_norm: Optional[torch.Tensor]
    lam: float
    o: torch.Tensor

    def tensors(self):
        return [t for t in (self.proj, self.q_norm, self.k_norm, self.o) if t is not None]


@dataclass
class PostBlockWeights:
    """One block with the norm on each sublayer's output: ``canon1`` / ``canon2`` [W, taps] the input convolutions of
    the mixer and the feed-forward, ``norm1`` / ``norm2`` [W], ``dwa`` fp32 [layer + 2] the weights of the depth
    average that leaves the layer (or None)."""
    norm1: torch.Tensor
    norm2: Optional[torch.Tensor]
    canon1: Optional[torch.Tensor]
    canon2: Optional[torch.Tensor]
    dwa: Optional[torch.Tensor]
    mix: object
    mlp: Optional[DenseMLPWeights]

    def tensors(self):
        out = [self.norm1] + self.mix.tensors()
        for t in (self.norm2, self.canon1, self.canon2, self.dwa):
            if t is not None:
                out.append(t)
        if self.mlp is not None:
            out += self.mlp.tensors()
        return out


def lamisun_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names of a Lamisun config and their shapes."""
    W = cfg.hidden_size
    out = {"embed": (cfg.vocab_size, W), "final.norm": (W,), "head": (cfg.vocab_size, W)}
    if cfg.bigram is not None:
        out["bigram"] = (cfg.bigram.buckets + 1, W)
    for i, spec in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", spec.mixer
        out[p + "norm1"] = (W,)
        if cfg.canon_taps:
            out[p + "canon1"] = (W, cfg.canon_taps)
        if m.kind == "latent_attention":
            out.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), W), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                        p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                        p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.o": (W, m.heads * m.vdim)})
            if m.gate:
                out[p + "mix.g"] = (m.heads * m.vdim, W)
        else:
            out.update({p + "mix.q": (m.heads * 2 * m.dim, W), p + "mix.k": (m.kv_heads * 2 * m.dim, W),
                        p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.o": (W, m.heads * m.vdim)})
            if m.qk_norm:
                out.update({p + "mix.q.norm": (m.dim,), p + "mix.k.norm": (m.dim,)})
            out.update({p + "mix." + n: (m.dim,) for n in ("lq1", "lk1", "lq2", "lk2")})
        if spec.mlp is not None:
            out.update({p + "norm2": (W,), p + "mlp.up": (spec.mlp.ff, W), p + "mlp.down": (W, spec.mlp.ff),
                        p + "mlp.act": (2,)})
            if cfg.canon_taps and cfg.canon_ffn:
                out[p + "canon2"] = (W, cfg.canon_taps)
        if cfg.depth_average:
            out[p + "dwa"] = (i + 2,)
    return out


def _lamisun_finish(cfg: ModelConfig, get, device, dtype) -> ModelWeights:
    """``get(name)`` returns the checkpoint tensor of that name (CPU). Shapes are checked against the config. Every
    input projection of a mixer becomes one matrix (latent attention: q | down-projection | gate; differential
    attention: q | k | v); numbers that are fixed once the weights are known (the second map's weight, the
    activation's two coefficients, the rotation's angular steps) are formed here, in fp32."""
    shapes = lamisun_shapes(cfg)

    def g(name):
        t = get(name)
        if tuple(t.shape) != shapes[name]:
            raise ValueError(f"{name} has shape {tuple(t.shape)}, the config says {shapes[name]}")
        return t

    def dev(t, dt=dtype):
        return None if t is None else t.to(device=device, dtype=dt).contiguous()

    def f32(t):
        return dev(t, torch.float32)

    def softplus(z: float) -> float:
        return float(torch.nn.functional.softplus(torch.tensor(z, dtype=torch.float32), threshold=80.0))
    layers = []
    for i, spec in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", spec.mixer
        if m.kind == "latent_attention":
            parts = [("q", g(p + "mix.q")), ("dkv", g(p + "mix.dkv"))]
            if m.gate:
                parts.append(("g", g(p + "mix.g")))
            qc, cols = _cat_rows(parts)
            freqs = None
            if m.rot_dim:
                freqs = f32(torch.tensor([m.rot.base ** (-2.0 * j / m.rot.dims) for j in range(m.rot.dims // 2)],
                                         dtype=torch.float64))
            mix = LatentAttnWeights(
                qc=dev(qc), own_kv=True, kv_norm=dev(g(p + "mix.dkv.norm")),
                uk_t=dev(_heads_t(g(p + "mix.uk"), m.heads, m.dim, m.kv_rank, i)), uv=dev(g(p + "mix.uv")),
                o=dev(g(p + "mix.o")), freqs=freqs, gate_col=cols.get("g"),
                rot_key=(m.rot.dims, m.rot.base) if m.rot_dim else None)
        else:
            proj, cols = _cat_rows([("q", g(p + "mix.q")), ("k", g(p + "mix.k")), ("v", g(p + "mix.v"))])
            lq1, lk1, lq2, lk2 = (g(p + "mix." + n).float() for n in ("lq1", "lk1", "lq2", "lk2"))
            lam = float(torch.exp((lq1 * lk1).sum()) - torch.exp((lq2 * lk2).sum()) + torch.tensor(m.diff))
            mix = DiffAttnWeights(dev(proj), cols, dev(g(p + "mix.q.norm")) if m.qk_norm else None,
                                  dev(g(p + "mix.k.norm")) if m.qk_norm else None, lam, dev(g(p + "mix.o")))
        mlp = None
        if spec.mlp is not None:
            a = g(p + "mlp.act").float()
            mlp = DenseMLPWeights(dev(g(p + "mlp.up")), dev(g(p + "mlp.down")),
                                  (softplus(float(a[0])), 0.5 + softplus(float(a[1]))))
        canon = bool(cfg.canon_taps)
        layers.append(PostBlockWeights(
            dev(g(p + "norm1")), dev(g(p + "norm2")) if mlp is not None else None,
            dev(g(p + "canon1")) if canon else None,
            dev(g(p + "canon2")) if canon and cfg.canon_ffn and mlp is not None else None,
            f32(g(p + "dwa")) if cfg.depth_average else None, mix, mlp))
    vp = math.ceil(cfg.vocab_size / 16) * 16
    head = torch.zeros(vp, cfg.hidden_size, dtype=dtype, device=device)
    head[:cfg.vocab_size].copy_(g("head").to(device=device, dtype=dtype))
    extra = {"bigram": dev(g("bigram"))} if cfg.bigram is not None else {}
    return ModelWeights(wte=dev(g("embed")), wpe=None, layers=layers, lnf_w=dev(g("final.norm")), lnf_b=None,
                        head=Linear(head), extra=extra)


def load_lamisun_weights(cfg: ModelConfig, reader, device="cpu", dtype=torch.bfloat16) -> ModelWeights:
    return _lamisun_finish(cfg, lambda n: reader.get(n), device, dtype)


def _lamisun_random(cfg: ModelConfig, seed: int, device="cpu"):
    import zlib

    shapes = lamisun_shapes(cfg)

    def get(name: str) -> torch.Tensor:
        gen = torch.Generator(device=device)
        gen.manual_seed((seed * 1000003 + zlib.crc32(name.encode())) & 0x7FFFFFFF)
        shp = shapes[name]
        t = torch.randn(*shp, generator=gen, dtype=torch.float32, device=device)
        last = name.split(".")[-1]
        if last.startswith("norm") or name == "final.norm":
            t = 1.0 + 0.1 * t
        elif last == "dwa":  # mostly the layer's own result, a little of every earlier one
            t = 0.1 * t
            t[-1] += 1.0
        elif last in ("canon1", "canon2"):
            t = t * shp[1] ** -0.5
        elif last in ("lq1", "lk1", "lq2", "lk2"):
            t = 0.4 * t
        elif last == "act":
            t = 0.5 * t
        elif name == "embed":
            t = t / max(cfg.embedding_scale, 1e-6)
        elif len(shp) == 2 and name != "bigram":
            t = t * shp[1] ** -0.5
        return t.to(torch.bfloat16).float()
    return get


def random_lamisun_weights(cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, seed: int = 0) -> ModelWeights:
    """Random-init weights of a Lamisun config (values rounded to bf16, so a bf16 and an fp32 run hold the same
    model): projections ~ N(0, 1 / fan_in), norm weights around one, depth averages around the plain stack."""
    gen = device if torch.device(device).type == "cuda" else "cpu"  # large models: draw on the GPU
    return _lamisun_finish(cfg, _lamisun_random(cfg, seed, gen), device, dtype)


def lamisun_state_dict(cfg: ModelConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """The random weights of :func:`random_lamisun_weights` under their checkpoint names (bf16; tests, examples)."""
    get = _lamisun_random(cfg, seed)
    return {n: get(n).to(torch.bfloat16) for n in lamisun_shapes(cfg)}


# ------------------------------------------------------------------------------ sandwich-normed per-layer designs (Fizelix)
@dataclass
class PoolAttnWeights:
    """Windowed sigmoid attention with pooled blocks: ``proj`` [q | k | v | sublayer gate rows padded to 8, W] (one
    GEMM), ``cols`` the first row of each part (``rg``: the gate logits of the block's gated residual); ``pb`` fp32
    [heads] the per-head score bias; ``freqs`` fp32 [rot.dims / 2] the pairs' angular steps per position (None: no
    rotation), ``rot_key`` (dims, base): layers with the same rotation share a step's angles; ``o`` [W, heads * vdim]."""
    proj: torch.Tensor
    cols: Dict[str, int]
    pb: torch.Tensor
    freqs: Optional[torch.Tensor]
    rot_key: Optional[tuple]
    o: torch.Tensor

    def tensors(self):
        return [t for t in (self.proj, self.pb, self.freqs, self.o) if t is not None]


@dataclass
class SSDWeights:
    """State-space mixer: ``proj`` [z | x | B | C | dt | sublayer gate rows padded to 8, W] (one GEMM), ``cols`` the
    first row of z, xbc (x, B, C side by side: one convolution), dt and rg; ``conv`` [channels, taps] with bias
    ``conv_b``; ``dt_bias``, ``A_log``, ``D`` fp32 [heads]; ``norm`` [heads * vdim]; ``o`` [W, heads * vdim]."""
    proj: torch.Tensor
    cols: Dict[str, int]
    conv: torch.Tensor
    conv_b: torch.Tensor
    dt_bias: torch.Tensor
    A_log: torch.Tensor
    D: torch.Tensor
    norm: torch.Tensor
    o: torch.Tensor

    def tensors(self):
        return [self.proj, self.conv, self.conv_b, self.dt_bias, self.A_log, self.D, self.norm, self.o]


@dataclass
class SandwichBlockWeights:
    """One block normed on both sides of its sublayers, x <- x + post * rms_norm(sigmoid(W_g h + b) * sublayer(h)), h =
    rms_norm(x) * norm. All vectors fp32: ``norm1`` / ``norm2``; ``post1`` / ``post2`` = the output norm's weight times
    the layer scale; ``rg1_b`` / ``rg2_b`` the gates' biases (the gates' matrices ride in the sublayers' first
    GEMMs: ``mix.cols["rg"]``, ``rg2_col``). Token input: ``side_gate`` [d, W], ``side_proj`` [W, d] in the storage
    type, ``side_norm`` fp32 [W], ``side_col`` the layer's first column in the token table."""
    norm1: torch.Tensor
    post1: torch.Tensor
    rg1_b: torch.Tensor
    mix: object
    norm2: Optional[torch.Tensor] = None
    post2: Optional[torch.Tensor] = None
    rg2_b: Optional[torch.Tensor] = None
    rg2_col: int = 0
    mlp: Optional[object] = None
    side_gate: Optional[torch.Tensor] = None
    side_proj: Optional[torch.Tensor] = None
    side_norm: Optional[torch.Tensor] = None
    side_col: int = 0

    def tensors(self):
        out = [self.norm1, self.post1, self.rg1_b] + self.mix.tensors()
        for t in (self.norm2, self.post2, self.rg2_b, self.side_gate, self.side_proj, self.side_norm):
            if t is not None:
                out.append(t)
        if self.mlp is not None:
            out += self.mlp.tensors()
        return out


def fizelix_shapes(cfg: ModelConfig) -> Dict[str, tuple]:
    """Checkpoint tensor names of a Fizelix config and their shapes."""
    W, L = cfg.hidden_size, len(cfg.layer_specs)
    out = {"embed": (cfg.vocab_size, W), "final.norm": (W,), "head": (cfg.vocab_size, W)}
    d = cfg.token_side_dim
    if d:
        out["side.embed"] = (cfg.vocab_size, L * d)
    for i, spec in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", spec.mixer
        for n in ("norm1", "norm1b", "ls1", "rg1.b"):
            out[p + n] = (W,)
        out[p + "rg1"] = (W, W)
        if m.kind == "pool_attention":
            out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.kv_heads * m.dim, W),
                        p + "mix.v": (m.kv_heads * m.vdim, W), p + "mix.pb": (m.heads,),
                        p + "mix.o": (W, m.heads * m.vdim)})
        else:
            C = m.conv_channels
            out.update({p + "mix.in": (2 * m.inner + 2 * m.groups * m.state + m.heads, W), p + "mix.conv": (C, m.conv),
                        p + "mix.conv.b": (C,), p + "mix.dt_bias": (m.heads,), p + "mix.A_log": (m.heads,),
                        p + "mix.D": (m.heads,), p + "mix.norm": (m.inner,), p + "mix.o": (W, m.inner)})
        f = spec.mlp
        if f is not None:
            for n in ("norm2", "norm2b", "ls2", "rg2.b"):
                out[p + n] = (W,)
            out[p + "rg2"] = (W, W)
            if f.kind == "dense":
                out.update({p + "mlp.gate": (f.ff, W), p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff)})
            else:
                out[p + "mlp.router"] = (f.experts, W)
                for k in range(f.experts):
                    out.update({f"{p}mlp.e{k}.gate": (f.expert.ff, W), f"{p}mlp.e{k}.up": (f.expert.ff, W),
                                f"{p}mlp.e{k}.down": (W, f.expert.ff)})
                if f.shared is not None:
                    out.update({p + "mlp.shared.gate": (f.shared.ff, W), p + "mlp.shared.up": (f.shared.ff, W),
                                p + "mlp.shared.down": (W, f.shared.ff)})
        if d:
            out.update({p + "side.gate": (d, W), p + "side.proj": (W, d), p + "side.norm": (W,)})
    return out


def _fizelix_finish(cfg: ModelConfig, get, device, dtype) -> ModelWeights:
    """``get(name)`` returns the checkpoint tensor of that name (CPU). Shapes are checked against the config. Every
    sublayer's first GEMM also carries the matrix of the sublayer's output gate (attention: q | k | v | gate; state
    space: in | gate; dense feed-forward: gate | up | gate of the residual; experts: beside the shared expert's
    gate | up, or alone). Norm weights, layer scales and biases are kept in fp32; the output norm's weight and the
    layer scale become one vector, the final norm's weight carries the logit scale."""
    shapes = fizelix_shapes(cfg)

    def g(name):
        t = get(name)
        if tuple(t.shape) != shapes[name]:
            raise ValueError(f"{name} has shape {tuple(t.shape)}, the config says {shapes[name]}")
        return t

    def dev(t, dt=dtype):
        return None if t is None else t.to(device=device, dtype=dt).contiguous()

    def f32(t):
        return dev(t.float(), torch.float32)
    d = cfg.token_side_dim
    layers = []
    for i, spec in enumerate(cfg.layer_specs):
        p, m = f"l{i}.", spec.mixer
        if m.kind == "pool_attention":
            proj, cols = _cat_rows([("q", g(p + "mix.q")), ("k", g(p + "mix.k")), ("v", g(p + "mix.v")),
                                    ("rg", g(p + "rg1"))])
            freqs = None
            if m.rot is not None:
                freqs = f32(torch.tensor([m.rot.base ** (-2.0 * j / m.rot.dims) for j in range(m.rot.dims // 2)],
                                         dtype=torch.float64))
            mix = PoolAttnWeights(dev(proj), cols, f32(g(p + "mix.pb")), freqs,
                                  (m.rot.dims, m.rot.base) if m.rot is not None else None, dev(g(p + "mix.o")))
        else:
            proj, cols = _cat_rows([("z", g(p + "mix.in")), ("rg", g(p + "rg1"))])
            cols["xbc"] = m.inner
            cols["dt"] = 2 * m.inner + 2 * m.groups * m.state
            mix = SSDWeights(dev(proj), cols, dev(g(p + "mix.conv")), dev(g(p + "mix.conv.b")),
                             f32(g(p + "mix.dt_bias")), f32(g(p + "mix.A_log")), f32(g(p + "mix.D")),
                             dev(g(p + "mix.norm")), dev(g(p + "mix.o")))
        blk = SandwichBlockWeights(f32(g(p + "norm1")), f32(g(p + "norm1b").float() * g(p + "ls1").float()),
                                   f32(g(p + "rg1.b")), mix)
        f = spec.mlp
        if f is not None:
            blk.norm2, blk.rg2_b = f32(g(p + "norm2")), f32(g(p + "rg2.b"))
            blk.post2 = f32(g(p + "norm2b").float() * g(p + "ls2").float())
            if f.kind == "dense":
                gu, cols = _cat_rows([("g", g(p + "mlp.gate")), ("u", g(p + "mlp.up")), ("rg", g(p + "rg2"))])
                blk.mlp, blk.rg2_col = DenseMLPWeights(dev(gu), dev(g(p + "mlp.down"))), cols["rg"]
            else:
                E, q = f.experts, p + "mlp."
                parts = [("rg", g(p + "rg2"))]
                if f.shared is not None:
                    parts = [("g", g(q + "shared.gate")), ("u", g(q + "shared.up"))] + parts
                sgu, cols = _cat_rows(parts)
                blk.mlp = MoEWeights(
                    router=dev(g(q + "router")), correction=None,
                    gate=dev(torch.stack([g(f"{q}e{k}.gate") for k in range(E)])),
                    up=dev(torch.stack([g(f"{q}e{k}.up") for k in range(E)])),
                    down=dev(torch.stack([g(f"{q}e{k}.down") for k in range(E)])),
                    shared_gu=dev(sgu), shared_down=dev(g(q + "shared.down")) if f.shared is not None else None)
                blk.rg2_col = cols["rg"]
        if d:
            blk.side_gate, blk.side_proj = dev(g(p + "side.gate")), dev(g(p + "side.proj"))
            blk.side_norm, blk.side_col = f32(g(p + "side.norm")), i * d
        layers.append(blk)
    vp = math.ceil(cfg.vocab_size / 16) * 16
    head = torch.zeros(vp, cfg.hidden_size, dtype=dtype, device=device)
    head[:cfg.vocab_size].copy_(g("head").to(device=device, dtype=dtype))
    extra = {"side": dev(g("side.embed"))} if d else {}
    return ModelWeights(wte=dev(g("embed")), wpe=None, layers=layers,
                        lnf_w=f32(g("final.norm").float() * cfg.logit_scale), lnf_b=None, head=Linear(head), extra=extra)


def load_fizelix_weights(cfg: ModelConfig, reader, device="cpu", dtype=torch.bfloat16) -> ModelWeights:
    return _fizelix_finish(cfg, lambda n: reader.get(n), device, dtype)


def _fizelix_random(cfg: ModelConfig, seed: int, device="cpu"):
    import zlib

    shapes = fizelix_shapes(cfg)

    def get(name: str) -> torch.Tensor:
        gen = torch.Generator(device=device)
        gen.manual_seed((seed * 1000003 + zlib.crc32(name.encode())) & 0x7FFFFFFF)
        shp = shapes[name]
        t = torch.randn(*shp, generator=gen, dtype=torch.float32, device=device)
        last = name.split(".")[-1]
        if name.endswith((".rg1.b", ".rg2.b", ".conv.b")):
            t = 0.3 * t
        elif last.startswith("norm") or name == "final.norm":
            t = 1.0 + 0.1 * t
        elif last in ("ls1", "ls2"):
            t = 0.5 + 0.1 * t
        elif last == "A_log":
            t = 0.5 * t - 0.5
        elif last in ("dt_bias", "pb"):
            t = 0.5 * t - (1.0 if last == "pb" else 0.0)
        elif last == "D":
            t = 1.0 + 0.2 * t
        elif last == "conv":
            t = t * shp[1] ** -0.5
        elif name == "embed":
            t = t / max(cfg.embedding_scale, 1e-6)
        elif len(shp) == 2 and name != "side.embed":
            t = t * shp[1] ** -0.5
        return t.to(torch.bfloat16).float()
    return get


def random_fizelix_weights(cfg: ModelConfig, device="cpu", dtype=torch.bfloat16, seed: int = 0) -> ModelWeights:
    """Random-init weights of a Fizelix config (values rounded to bf16, so a bf16 and an fp32 run hold the same
    model): projections ~ N(0, 1 / fan_in), norm weights around one, layer scales around one half."""
    gen = device if torch.device(device).type == "cuda" else "cpu"  # large models: draw on the GPU
    return _fizelix_finish(cfg, _fizelix_random(cfg, seed, gen), device, dtype)


def fizelix_state_dict(cfg: ModelConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
    """The random weights of :func:`random_fizelix_weights` under their checkpoint names (bf16; tests, examples)."""
    get = _fizelix_random(cfg, seed)
    return {n: get(n).to(torch.bfloat16) for n in fizelix_shapes(cfg)}
