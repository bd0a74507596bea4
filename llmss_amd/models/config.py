"""Architecture description shared by every model family.

The reference builds each family from a ``transformers.PretrainedConfig`` subclass and
``PreTrainedModel`` glue (``gptj_modeling.py:320-354``, ``gpt_bigcode_modeling.py:417-462``).
Here a single flat dataclass captures everything the native decoder needs; it is parsed
from a HF ``config.json`` (no ``transformers`` import on the hot path) or built from a named
preset for synthetic/random-init runs (bench, smoke tests).

Families (``MODEL_REGISTRY`` keys, reference ``custom_modeling/__init__.py:4-7`` had only
``gptj`` and ``gpt_bigcode``):

* ``gpt2``        - LayerNorm, learned positions, Conv1D fused c_attn, GELU-tanh, tied head.
* ``gptj``        - LayerNorm, *parallel* residual block, interleaved partial RoPE,
                    separate q/k/v without bias, lm_head with bias (``gptj_modeling.py``).
* ``gpt_bigcode`` - LayerNorm, learned positions, MQA (or MHA) fused c_attn, tied head
                    (``gpt_bigcode_modeling.py``).
* ``llama``       - RMSNorm, half-rotate RoPE, GQA, SwiGLU, untied head.
* ``timisun``     - per-layer description (``layer_specs``): parallel blocks over an fp32 residual, latent
                    attention without positions (sliding window, latent rows shared between layers),
                    mixture-of-experts feed-forward with a shared expert, scaled embedding, tied head.
* ``babotar``     - per-layer description: sequential pre-norm blocks (bias-free layer norm) over one or several
                    fp32 residual streams, optional causal input convolution, mixers ``parallel`` (sink attention
                    beside a gated delta rule) and ``lightning`` (decay linear attention), gated tanh-GELU
                    feed-forward, learned positions, untied head.
* ``lamisun``     - per-layer description: sequential blocks whose norm sits on each sublayer's OUTPUT
                    (x <- x + norm(sublayer(x + conv(x)))), a causal input convolution before both sublayers, the
                    layers' results averaged over depth with learned weights, a hashed bigram row added to the
                    embedding; mixers ``latent_attention`` (with a rotated key part shared by the heads and an output
                    gate) and ``attention`` (two softmax maps subtracted, chunked mask, query / key norm);
                    plain feed-forward with the xIELU activation, untied head.
* ``fizelix``     - per-layer description: blocks normed before AND after each sublayer, the sublayer's result gated
                    by sigmoid(W h + b) and scaled per channel, a per-layer token input after the feed-forward, a run
                    of layers repeated with the same weights (the embedding added again before each repeat); mixers
                    ``pool_attention`` (sigmoid-weighted sliding window plus mean-pooled blocks of older tokens,
                    neighbour-pair rotation) and ``mamba2`` (state-space duality: decayed matrix state per head, short
                    convolution, gate before a grouped norm); feed-forward dense SiLU-gated or mixture of experts whose
                    sigmoid score multiplies the expert's input; scaled logits, untied head.
"""
from __future__ import annotations

import json
import math
import os
from dataclasses import asdict, dataclass, field, replace
from typing import Any, Dict, List, Optional


@dataclass
class MixerSpec:
    """One layer's token mixer. ``latent_attention``: ``heads`` heads of ``dim`` query/key and ``vdim`` value
    dimensions over a cached latent row of ``kv_rank`` numbers; ``window`` > 0 limits a position to itself and the
    ``window - 1`` positions before it (0 = every earlier position); ``kv_from`` = index of the layer whose cached
    latent rows this layer reads instead of projecting its own."""
    kind: str
    heads: int
    dim: int
    vdim: int
    kv_rank: int
    scale: float
    window: int = 0
    kv_from: Optional[int] = None
    # ``rot_dim`` > 0: every query head carries ``rot_dim`` more numbers after its ``dim`` and the down-projection
    # ``rot_dim`` more rows after the latent - one key part shared by all heads - both turned by ``rot`` (pairs of
    # neighbours, the first ``rot.dims`` <= rot_dim numbers; the rest pass unchanged) and multiplied into the score
    # beside the latent part; the rotated key part is cached with the latent
    rot_dim: int = 0
    rot: Optional["RotarySpec"] = None
    gate: bool = False  # the concatenated heads are multiplied by sigmoid(W_g h) before the output projection


@dataclass
class ExpertSpec:
    ff: int
    limit: float = 0.0


@dataclass
class MoESpec:
    """Mixture-of-experts feed-forward: ``experts`` experts of which each token uses ``top``; ``shared`` runs for
    every token."""
    experts: int
    top: int
    expert: ExpertSpec
    shared: Optional[ExpertSpec] = None
    kind: str = "moe"
    act: str = "glu_clamp"  # "glu_clamp": g sigmoid(1.702 g) (u + 1) with clamps; "silu": silu(g) u, no clamps
    normalize: bool = True  # the chosen scores are divided by their sum
    weight_input: bool = False  # the score multiplies the expert's input (sum_e expert_e(w_e h)), not its output


@dataclass
class RotarySpec:
    """Rotary positions on the first ``dims`` dimensions of a head, dimension i paired with i + dims / 2, frequency
    base^(-2 i / dims); ``scaling`` = (factor, original length, fast turns, slow turns) blends the frequencies
    between the two turn counts towards f / factor and scales cos and sin by 0.1 ln(factor) + 1."""
    dims: int
    base: float
    scaling: Optional[tuple] = None
    pairs: str = "half"  # "half": i with i + dims / 2; "neighbours": 2i with 2i + 1


@dataclass
class SinkAttnSpec:
    """Softmax attention over a paged key/value cache: ``heads`` query heads on ``kv_heads`` key/value heads, key
    size ``dim``, value size ``vdim``; scores times ``scale``, soft-capped when ``softcap`` > 0; one unit added to
    the softmax denominator (a sink); ``talk``: the heads' weights are mixed by an [heads, heads] matrix; ``bias``:
    the q / k / v projections have biases."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    softcap: float = 0.0
    rot: Optional[RotarySpec] = None
    talk: bool = False
    bias: bool = False
    kind: str = "sink_attention"


@dataclass
class DiffAttnSpec:
    """Differential softmax attention over a paged key/value cache: every query head and every key head holds two
    maps of ``dim`` numbers that attend separately over the same values (``vdim`` per key/value head); per head
    o = a1 - lambda a2, divided by its root mean square and multiplied by 1 - ``diff``. lambda is one number of the
    layer: exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff``. ``qk_norm``: queries and keys are RMS-normed per head and map
    with a learned weight; ``chunk`` > 0: a position sees the earlier positions of its own block of ``chunk``
    positions only (0: all earlier positions)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    diff: float
    chunk: int = 0
    qk_norm: bool = True
    kind: str = "attention"


@dataclass
class PoolAttnSpec:
    """Sigmoid-weighted attention over a paged key/value cache, no softmax: ``heads`` query heads on ``kv_heads``
    key/value heads; the weight of a visible key is sigmoid(q . k * scale + bias[head]), weights are not normalised.
    Position i sees the positions j with 0 <= i - j < ``window`` (0: all earlier ones) and, with ``pool`` > 0, one
    mean key and mean value for every block of ``pool`` positions that ends at or before i - window. ``rot``:
    rotation of neighbouring pairs of the first ``rot.dims`` numbers of every query and key head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0
    pool: int = 0
    rot: Optional[RotarySpec] = None
    kind: str = "pool_attention"


@dataclass
class SSDSpec:
    """State-space mixer with a scalar decay per head and token: a matrix state [state, vdim] per head, ``groups``
    input / output vectors (B, C) shared by heads / groups heads each, x | B | C through a causal convolution of
    ``conv`` taps with bias and SiLU; the heads' outputs are gated by silu(z) and then RMS-normed in ``norm_groups``
    equal parts."""
    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1
    kind: str = "mamba2"

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.inner + 2 * self.groups * self.state


@dataclass
class BigramSpec:
    """A second embedding table of ``buckets`` + 1 rows: row (previous * mul_prev + current * mul_cur) mod buckets is
    added to a token's embedding, the last row for a sequence's first token."""
    buckets: int
    mul_prev: int
    mul_cur: int


@dataclass
class DeltaSpec:
    """Gated delta rule: a matrix state [dim, vdim] per head, ``kv_heads`` query/key heads shared by ``heads`` value
    heads, q / k / v through a short causal convolution of ``conv`` taps."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    kind: str = "gated_delta"


@dataclass
class DecaySpec:
    """Linear attention with a constant decay per head over a matrix state [dim, vdim]."""
    heads: int
    dim: int
    vdim: int
    decay: tuple = ()
    kind: str = "lightning"


@dataclass
class ParallelMixerSpec:
    """Two mixers reading the same input; the result is left_scale * left + right_scale * right."""
    left: SinkAttnSpec
    right: DeltaSpec
    left_scale: float = 1.0
    right_scale: float = 1.0
    kind: str = "parallel"


@dataclass
class DenseMLPSpec:
    """Feed-forward down(act(gate h) * (up h)), or, ``gated`` false, down(act(up h)). ``act``: ``gelu_tanh``,
    ``silu`` or ``xielu`` (two learned numbers per layer)."""
    ff: int
    act: str = "gelu_tanh"
    kind: str = "dense"
    gated: bool = True


@dataclass
class LayerSpec:
    mixer: Any
    mlp: Optional[Any] = None


@dataclass
class ModelConfig:
    model_type: str
    vocab_size: int
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    max_position_embeddings: int
    norm: str = "layernorm"  # "layernorm" | "rmsnorm"
    norm_eps: float = 1e-5
    activation: str = "gelu_tanh"  # "gelu_tanh" | "gelu" | "silu_glu" | "relu"
    position: str = "learned"  # "learned" | "rope"
    rope_style: str = "neox"  # "neox" (half rotate) | "gptj" (interleaved pairs)
    rotary_dim: int = 0
    rope_theta: float = 10000.0
    parallel_block: bool = False  # GPT-J: attn and mlp read the same LN output
    tie_word_embeddings: bool = False
    qkv_bias: bool = False
    out_bias: bool = False
    mlp_bias: bool = False
    lm_head_bias: bool = False
    conv1d_weights: bool = False  # GPT-2 stores [in, out] Conv1D weights
    fused_qkv_name: Optional[str] = None  # checkpoint tensor name of the fused c_attn, if any
    bos_token_id: Optional[int] = None
    eos_token_id: Optional[int] = None
    pad_token_id: Optional[int] = None
    extra: Dict[str, Any] = field(default_factory=dict)
    # per-layer designs (layers that differ from each other): one LayerSpec per layer; None for the uniform families
    layer_specs: Optional[List[LayerSpec]] = None
    embedding_scale: float = 1.0  # the embedding row is multiplied by this
    norm_offset: float = 0.0  # norm weights are stored as (w - offset): 1.0 = stored around zero
    residual_fp32: bool = False  # the residual stream is kept and summed in fp32
    # sequential per-layer blocks (x <- x + c * mixer(norm1(x)); x <- x + c * ffn(norm2(x))):
    streams: int = 0  # > 0: that many residual streams with learned read / write / mix weights per sublayer
    residual_mult: float = 1.0  # c above
    canon_taps: int = 0  # > 0: the mixer's input h becomes h + causal_conv(h) over that many taps
    # blocks whose norm sits on the sublayer's output (x <- x + norm(sublayer(x))); the sublayers read x itself
    post_norm: bool = False
    canon_ffn: bool = False  # the feed-forward's input goes through an input convolution of its own as well
    depth_average: bool = False  # what leaves layer i is a learned weighted sum of the results of layers <= i
    bigram: Optional[BigramSpec] = None
    # blocks normed on both sides of a sublayer: x <- x + scale * norm_b(gate * sublayer(norm_a(x))), gate =
    # sigmoid(W norm_a(x) + b) per channel
    sandwich: bool = False
    token_side_dim: int = 0  # > 0: after the feed-forward a layer adds a normed projection of its slice of a second token table
    loop: Optional[tuple] = None  # (start, stop, times): layers start .. stop - 1 run ``times`` times in a row
    logit_scale: float = 1.0

    def layer_runs(self) -> List[int]:
        """Layer index of every layer run, in order: a looped stretch repeats with the same weights, each pass with
        cache and state of its own."""
        n = len(self.layer_specs) if self.layer_specs else self.num_layers
        if not self.loop or self.loop[2] <= 1:
            return list(range(n))
        a, b, times = self.loop
        return list(range(a)) + list(range(a, b)) * times + list(range(b, n))

    # ---------------------------------------------------------------- derived
    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def gated_mlp(self) -> bool:
        return self.activation == "silu_glu"

    @property
    def n_positions(self) -> int:  # reference name (generate.py:60)
        return self.max_position_embeddings

    def num_params(self) -> int:
        h, f, v = self.hidden_size, self.intermediate_size, self.vocab_size
        if self.layer_specs and self.model_type in ("babotar", "lamisun", "fizelix"):
            from .weights import babotar_shapes, fizelix_shapes, lamisun_shapes

            shapes = {"babotar": babotar_shapes, "lamisun": lamisun_shapes, "fizelix": fizelix_shapes}[
                self.model_type](self)
            return sum(math.prod(shp) for shp in shapes.values())
        if self.layer_specs:
            n = v * h + h
            for s in self.layer_specs:
                m = s.mixer
                n += h + m.heads * m.dim * h + (m.kv_rank * (h + 1) if m.kv_from is None else 0)
                n += m.heads * (m.dim + m.vdim) * m.kv_rank + h * m.heads * m.vdim
                if s.mlp is not None:
                    n += s.mlp.experts * (h + 1 + 3 * h * s.mlp.expert.ff)
                    n += 3 * h * s.mlp.shared.ff if s.mlp.shared else 0
            return n
        attn = h * (self.q_size + 2 * self.kv_size) + self.q_size * h
        mlp = (3 if self.gated_mlp else 2) * h * f
        per_layer = attn + mlp + 4 * h
        emb = v * h + (self.max_position_embeddings * h if self.position == "learned" else 0)
        head = 0 if self.tie_word_embeddings else v * h
        return self.num_layers * per_layer + emb + head

    def to_dict(self) -> Dict[str, Any]:
        return asdict(self)

    # ---------------------------------------------------------------- parsing
    @classmethod
    def from_hf_dict(cls, d: Dict[str, Any]) -> "ModelConfig":
        mt = d.get("model_type")
        if mt is None and d.get("architecture") == "Timisun":
            return _timisun(cls, d)
        if mt is None and d.get("architecture") == "Babotar":
            return _babotar(cls, d)
        if mt is None and d.get("architecture") == "Lamisun":
            return _lamisun(cls, d)
        if mt is None and d.get("architecture") == "Fizelix":
            return _fizelix(cls, d)
        common = dict(
            bos_token_id=d.get("bos_token_id"),
            eos_token_id=_first(d.get("eos_token_id")),
            pad_token_id=d.get("pad_token_id"),
        )
        if mt == "gpt2":
            h, nh = d["n_embd"], d["n_head"]
            return cls(
                model_type="gpt2", vocab_size=d["vocab_size"], hidden_size=h, num_layers=d["n_layer"],
                num_heads=nh, num_kv_heads=nh, head_dim=h // nh,
                intermediate_size=d.get("n_inner") or 4 * h, max_position_embeddings=d["n_positions"],
                norm="layernorm", norm_eps=d.get("layer_norm_epsilon", 1e-5),
                activation=_act(d.get("activation_function", "gelu_new")), position="learned",
                tie_word_embeddings=d.get("tie_word_embeddings", True), qkv_bias=True, out_bias=True,
                mlp_bias=True, conv1d_weights=True, fused_qkv_name="c_attn", **common,
            )
        if mt == "gptj":
            h, nh = d["n_embd"], d["n_head"]
            hd = h // nh
            return cls(
                model_type="gptj", vocab_size=d["vocab_size"], hidden_size=h, num_layers=d["n_layer"],
                num_heads=nh, num_kv_heads=nh, head_dim=hd,
                intermediate_size=d.get("n_inner") or 4 * h, max_position_embeddings=d["n_positions"],
                norm="layernorm", norm_eps=d.get("layer_norm_epsilon", 1e-5),
                activation=_act(d.get("activation_function", "gelu_new")), position="rope",
                rope_style="gptj", rotary_dim=d.get("rotary_dim") or hd, parallel_block=True,
                tie_word_embeddings=d.get("tie_word_embeddings", False), qkv_bias=False, out_bias=False,
                mlp_bias=True, lm_head_bias=True, **common,
            )
        if mt == "gpt_bigcode":
            h, nh = d["n_embd"], d["n_head"]
            mq = d.get("multi_query", True)
            return cls(
                model_type="gpt_bigcode", vocab_size=d["vocab_size"], hidden_size=h, num_layers=d["n_layer"],
                num_heads=nh, num_kv_heads=1 if mq else nh, head_dim=h // nh,
                intermediate_size=d.get("n_inner") or 4 * h, max_position_embeddings=d["n_positions"],
                norm="layernorm", norm_eps=d.get("layer_norm_epsilon", 1e-5),
                activation=_act(d.get("activation_function", "gelu_pytorch_tanh")), position="learned",
                tie_word_embeddings=d.get("tie_word_embeddings", True), qkv_bias=True, out_bias=True,
                mlp_bias=True, fused_qkv_name="c_attn", **common,
            )
        if mt in ("llama", "mistral"):
            h, nh = d["hidden_size"], d["num_attention_heads"]
            hd = d.get("head_dim") or h // nh
            return cls(
                model_type="llama", vocab_size=d["vocab_size"], hidden_size=h, num_layers=d["num_hidden_layers"],
                num_heads=nh, num_kv_heads=d.get("num_key_value_heads") or nh, head_dim=hd,
                intermediate_size=d["intermediate_size"],
                max_position_embeddings=d.get("max_position_embeddings", 4096),
                norm="rmsnorm", norm_eps=d.get("rms_norm_eps", 1e-6), activation="silu_glu", position="rope",
                rope_style="neox", rotary_dim=hd, rope_theta=_rope_theta(d),
                tie_word_embeddings=d.get("tie_word_embeddings", False),
                qkv_bias=d.get("attention_bias", False), out_bias=d.get("attention_bias", False),
                mlp_bias=d.get("mlp_bias", False), **common,
            )
        raise ValueError(f"unsupported model_type {mt!r}; supported: gpt2, gptj, gpt_bigcode, llama")

    @classmethod
    def from_pretrained(cls, path: str) -> "ModelConfig":
        with open(os.path.join(path, "config.json")) as f:
            return cls.from_hf_dict(json.load(f))


def _timisun(cls, d: Dict[str, Any]) -> "ModelConfig":
    """``{"architecture": "Timisun", "vocab", "width", "embedding": {"scale"}, "norm": {"eps"}, "layers": [{"type",
    "mixer": {"heads", "dim", "vdim", "kv_rank", "scale", "mask": {"size"}, "kv_from"}, "mlp": {"kind": "moe",
    "router": {"experts", "top"}, "expert": {"ff", "limit"}, "shared": {"ff", "limit"}} | null}]}``."""
    specs: List[LayerSpec] = []
    for i, L in enumerate(d["layers"]):
        if L.get("type") != "latent_attention":
            raise ValueError(f"Timisun layer {i}: unsupported mixer type {L.get('type')!r}")
        m = L["mixer"]
        mask = m.get("mask") or {}
        kv_from = m.get("kv_from")
        mixer = MixerSpec("latent_attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]),
                          float(m["scale"]), int(mask.get("size") or 0), None if kv_from is None else int(kv_from))
        if mixer.kv_from is not None:
            j = mixer.kv_from
            if not 0 <= j < i or specs[j].mixer.kv_from is not None or specs[j].mixer.kv_rank != mixer.kv_rank:
                raise ValueError(f"Timisun layer {i}: kv_from {j} must name an earlier layer that projects its own "
                                 f"latent rows of the same rank")
        mlp = None
        f = L.get("mlp")
        if f is not None:
            if f.get("kind", "moe") != "moe":
                raise ValueError(f"Timisun layer {i}: unsupported feed-forward kind {f.get('kind')!r}")
            sh = f.get("shared")
            mlp = MoESpec(int(f["router"]["experts"]), int(f["router"]["top"]),
                          ExpertSpec(int(f["expert"]["ff"]), float(f["expert"]["limit"])),
                          None if sh is None else ExpertSpec(int(sh["ff"]), float(sh["limit"])))
            if not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"Timisun layer {i}: top {mlp.top} of {mlp.experts} experts")
        specs.append(LayerSpec(mixer, mlp))
    if not specs:
        raise ValueError("Timisun: no layers")
    return cls(
        model_type="timisun", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), num_layers=len(specs),
        num_heads=max(s.mixer.heads for s in specs), num_kv_heads=1, head_dim=max(s.mixer.kv_rank for s in specs),
        intermediate_size=max([s.mlp.expert.ff for s in specs if s.mlp] or [0]),
        max_position_embeddings=1 << 20,  # the design has no positional limit of its own
        norm="rmsnorm", norm_eps=float(d["norm"]["eps"]), activation="glu_clamp", position="none", rotary_dim=0,
        parallel_block=True, tie_word_embeddings=True, layer_specs=specs,
        embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), norm_offset=1.0, residual_fp32=True,
        bos_token_id=d.get("bos_token_id"), eos_token_id=_first(d.get("eos_token_id")),
        pad_token_id=d.get("pad_token_id"),
    )


def _babotar(cls, d: Dict[str, Any]) -> "ModelConfig":
    """``{"architecture": "Babotar", "vocab", "width", "max_positions", "norm": {"eps"}, "residual_mult", "streams",
    "canon": {"taps"}, "layers": [{"type": "lightning" | "parallel", "mixer": {...}, "mlp": {"kind": "dense", "ff"} |
    null}]}``. A lightning mixer gives heads, dim, vdim, decay; a parallel one ``left`` (heads, kv_heads, dim, vdim,
    scale, softcap, rot: {base, dims, scaling: {factor, original, fast, slow}}), ``right`` (heads, kv_heads, dim,
    vdim, conv), left_scale, right_scale. Keys that a config leaves out switch their mechanism off (no streams, no
    input convolution, no cap, no rotation, no frequency scaling); the head-mixing matrix and the q / k / v biases
    are found by their tensors at load."""
    specs: List[LayerSpec] = []
    for i, L in enumerate(d["layers"]):
        m, typ = L["mixer"], L.get("type")
        if typ == "lightning":
            mixer = DecaySpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), tuple(float(x) for x in m["decay"]))
            if len(mixer.decay) != mixer.heads:
                raise ValueError(f"Babotar layer {i}: {len(mixer.decay)} decays for {mixer.heads} heads")
        elif typ == "parallel":
            a, r = m["left"], m["right"]
            rot = None
            if a.get("rot"):
                sc = a["rot"].get("scaling")
                rot = RotarySpec(int(a["rot"]["dims"]), float(a["rot"]["base"]),
                                 None if not sc else (float(sc["factor"]), float(sc["original"]), float(sc["fast"]),
                                                      float(sc["slow"])))
                if rot.dims % 2 or rot.dims > int(a["dim"]):
                    raise ValueError(f"Babotar layer {i}: {rot.dims} rotary dimensions on heads of {a['dim']}")
            left = SinkAttnSpec(int(a["heads"]), int(a.get("kv_heads") or a["heads"]), int(a["dim"]), int(a["vdim"]),
                                float(a["scale"]) if "scale" in a else int(a["dim"]) ** -0.5,
                                float(a.get("softcap") or 0.0), rot, talk=True, bias=True)
            right = DeltaSpec(int(r["heads"]), int(r.get("kv_heads") or r["heads"]), int(r["dim"]), int(r["vdim"]),
                              int(r.get("conv") or 1))
            for nm, sp in (("left", left), ("right", right)):
                if sp.heads % sp.kv_heads:
                    raise ValueError(f"Babotar layer {i} {nm}: {sp.heads} heads on {sp.kv_heads} key heads")
            mixer = ParallelMixerSpec(left, right, float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))
        else:
            raise ValueError(f"Babotar layer {i}: unsupported mixer type {typ!r}")
        f, mlp = L.get("mlp"), None
        if f is not None:
            if f.get("kind", "dense") != "dense":
                raise ValueError(f"Babotar layer {i}: unsupported feed-forward kind {f.get('kind')!r}")
            mlp = DenseMLPSpec(int(f["ff"]))
        specs.append(LayerSpec(mixer, mlp))
    if not specs:
        raise ValueError("Babotar: no layers")
    heads = [s.mixer.left.heads if s.mixer.kind == "parallel" else s.mixer.heads for s in specs]
    return cls(
        model_type="babotar", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), num_layers=len(specs),
        num_heads=max(heads), num_kv_heads=1, head_dim=1,
        intermediate_size=max([s.mlp.ff for s in specs if s.mlp] or [0]),
        max_position_embeddings=int(d["max_positions"]), norm="layernorm", norm_eps=float(d["norm"]["eps"]),
        activation="gelu_tanh_glu", position="learned", rotary_dim=0, parallel_block=False,
        tie_word_embeddings=False, layer_specs=specs, residual_fp32=True, streams=int(d.get("streams") or 0),
        residual_mult=float(d.get("residual_mult", 1.0)), canon_taps=int((d.get("canon") or {}).get("taps") or 0),
        bos_token_id=d.get("bos_token_id"), eos_token_id=_first(d.get("eos_token_id")),
        pad_token_id=d.get("pad_token_id"),
    )


def _lamisun(cls, d: Dict[str, Any]) -> "ModelConfig":
    """``{"architecture": "Lamisun", "vocab", "width", "norm": {"eps"}, "canon": {"taps"}, "embedding": {"scale",
    "bigram": {"buckets", "mul_prev", "mul_cur"}}, "layers": [{"type": "latent_attention" | "attention", "mixer":
    {...}, "mlp": {"kind": "dense", "ff"} | null}]}``. A latent mixer gives heads, dim, rot_dim, vdim, kv_rank, scale,
    rot: {base, dims}; an attention mixer heads, kv_heads, dim, vdim, scale, diff, mask: {size}."""
    specs: List[LayerSpec] = []
    for i, L in enumerate(d["layers"]):
        m, typ = L["mixer"], L.get("type")
        if typ == "latent_attention":
            rd = int(m.get("rot_dim") or 0)
            rot = None
            if rd:
                rot = RotarySpec(int(m["rot"]["dims"]), float(m["rot"]["base"]), None, "neighbours")
                if rot.dims > rd or rot.dims % 2:
                    raise ValueError(f"Lamisun layer {i}: {rot.dims} rotary dimensions on a rotated part of {rd}")
            mixer = MixerSpec("latent_attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]), int(m["kv_rank"]),
                              float(m["scale"]), 0, None, rd, rot, True)
        elif typ == "attention":
            mixer = DiffAttnSpec(int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"]),
                                 float(m["scale"]), float(m["diff"]), int((m.get("mask") or {}).get("size") or 0))
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"Lamisun layer {i}: {mixer.heads} heads on {mixer.kv_heads} key heads")
        else:
            raise ValueError(f"Lamisun layer {i}: unsupported mixer type {typ!r}")
        f, mlp = L.get("mlp"), None
        if f is not None:
            if f.get("kind", "dense") != "dense":
                raise ValueError(f"Lamisun layer {i}: unsupported feed-forward kind {f.get('kind')!r}")
            mlp = DenseMLPSpec(int(f["ff"]), "xielu", gated=False)
        specs.append(LayerSpec(mixer, mlp))
    if not specs:
        raise ValueError("Lamisun: no layers")
    emb = d.get("embedding") or {}
    bg = emb.get("bigram")
    bigram = None if not bg else BigramSpec(int(bg["buckets"]), int(bg["mul_prev"]), int(bg["mul_cur"]))
    if bigram is not None and bigram.buckets < 1:
        raise ValueError("Lamisun: the bigram table needs at least one bucket")
    return cls(
        model_type="lamisun", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), num_layers=len(specs),
        num_heads=max(s.mixer.heads for s in specs), num_kv_heads=1, head_dim=1,
        intermediate_size=max([s.mlp.ff for s in specs if s.mlp] or [0]),
        max_position_embeddings=1 << 20,  # the design has no positional limit of its own
        norm="rmsnorm", norm_eps=float(d["norm"]["eps"]), activation="xielu", position="none", rotary_dim=0,
        parallel_block=False, tie_word_embeddings=False, layer_specs=specs, residual_fp32=True,
        embedding_scale=float(emb.get("scale", 1.0)), canon_taps=int((d.get("canon") or {}).get("taps") or 0),
        post_norm=True, canon_ffn=True, depth_average=True, bigram=bigram,
        bos_token_id=d.get("bos_token_id"), eos_token_id=_first(d.get("eos_token_id")),
        pad_token_id=d.get("pad_token_id"),
    )


def _fizelix(cls, d: Dict[str, Any]) -> "ModelConfig":
    """``{"architecture": "Fizelix", "vocab", "width", "norm": {"eps"}, "embedding": {"scale"}, "logit_scale",
    "token_side": {"dim"}, "loop": {"start", "stop", "times"}, "layers": [{"type": "attention" | "mamba2", "mixer":
    {...}, "mlp": {"kind": "dense", "ff"} | {"kind": "moe", "router": {"experts", "top"}, "expert": {"ff"}, "shared":
    {"ff"}} | null}]}``. An attention mixer gives heads, kv_heads, dim, vdim, scale, mask: {size, pool}, rot: {base,
    dims}; a mamba2 mixer heads, vdim, state, groups, conv, norm_groups. Keys a config leaves out switch their
    mechanism off (no loop, no token input, no rotation, no pooled blocks, no window, no shared expert)."""
    specs: List[LayerSpec] = []
    for i, L in enumerate(d["layers"]):
        m, typ = L["mixer"], L.get("type")
        if typ == "attention":
            rot = None
            if m.get("rot") and int(m["rot"].get("dims") or 0):
                rot = RotarySpec(int(m["rot"]["dims"]), float(m["rot"]["base"]), None, "neighbours")
                if rot.dims % 2 or rot.dims > int(m["dim"]):
                    raise ValueError(f"Fizelix layer {i}: {rot.dims} rotary dimensions on heads of {m['dim']}")
            mask = m.get("mask") or {}
            mixer = PoolAttnSpec(int(m["heads"]), int(m.get("kv_heads") or m["heads"]), int(m["dim"]), int(m["vdim"]),
                                 float(m["scale"]), int(mask.get("size") or 0), int(mask.get("pool") or 0), rot)
            if mixer.heads % mixer.kv_heads:
                raise ValueError(f"Fizelix layer {i}: {mixer.heads} heads on {mixer.kv_heads} key heads")
            if mixer.pool and not mixer.window:
                raise ValueError(f"Fizelix layer {i}: pooled blocks need a window")
        elif typ == "mamba2":
            mixer = SSDSpec(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups") or 1),
                            int(m.get("conv") or 1), int(m.get("norm_groups") or 1))
            if mixer.heads % mixer.groups or mixer.inner % mixer.norm_groups:
                raise ValueError(f"Fizelix layer {i}: {mixer.heads} heads in {mixer.groups} groups, "
                                 f"{mixer.inner} channels in {mixer.norm_groups} norm groups")
        else:
            raise ValueError(f"Fizelix layer {i}: unsupported mixer type {typ!r}")
        f, mlp = L.get("mlp"), None
        if f is not None:
            kind = f.get("kind", "dense")
            if kind == "dense":
                mlp = DenseMLPSpec(int(f["ff"]), "silu")
            elif kind == "moe":
                sh = f.get("shared")
                mlp = MoESpec(int(f["router"]["experts"]), int(f["router"]["top"]), ExpertSpec(int(f["expert"]["ff"])),
                              None if not sh else ExpertSpec(int(sh["ff"])), act="silu", normalize=False,
                              weight_input=True)
                if not 1 <= mlp.top <= mlp.experts:
                    raise ValueError(f"Fizelix layer {i}: top {mlp.top} of {mlp.experts} experts")
            else:
                raise ValueError(f"Fizelix layer {i}: unsupported feed-forward kind {kind!r}")
        specs.append(LayerSpec(mixer, mlp))
    if not specs:
        raise ValueError("Fizelix: no layers")
    loop = None
    lp = d.get("loop")
    if lp and int(lp.get("times", 1)) > 1:
        loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
        if not 0 <= loop[0] < loop[1] <= len(specs):
            raise ValueError(f"Fizelix: loop over layers {loop[0]} .. {loop[1] - 1} of {len(specs)}")
    ffs = [s.mlp.ff if s.mlp.kind == "dense" else s.mlp.expert.ff for s in specs if s.mlp]
    return cls(
        model_type="fizelix", vocab_size=int(d["vocab"]), hidden_size=int(d["width"]), num_layers=len(specs),
        num_heads=max(s.mixer.heads for s in specs), num_kv_heads=1, head_dim=1, intermediate_size=max(ffs or [0]),
        max_position_embeddings=1 << 20,  # the design has no positional limit of its own
        norm="rmsnorm", norm_eps=float(d["norm"]["eps"]), activation="silu_glu", position="none", rotary_dim=0,
        parallel_block=False, tie_word_embeddings=False, layer_specs=specs, residual_fp32=True,
        embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)), sandwich=True,
        token_side_dim=int((d.get("token_side") or {}).get("dim") or 0), loop=loop,
        logit_scale=float(d.get("logit_scale", 1.0)),
        bos_token_id=d.get("bos_token_id"), eos_token_id=_first(d.get("eos_token_id")),
        pad_token_id=d.get("pad_token_id"),
    )


def _first(x):
    if isinstance(x, (list, tuple)):
        return x[0] if x else None
    return x


def _act(name: str) -> str:
    name = name.lower()
    if name in ("gelu_new", "gelu_pytorch_tanh", "gelu_fast", "gelu_tanh"):
        return "gelu_tanh"
    if name in ("gelu",):
        return "gelu"
    if name in ("relu",):
        return "relu"
    if name in ("silu", "swish"):
        return "silu_glu"
    raise ValueError(f"unsupported activation {name}")


def _rope_theta(d: Dict[str, Any]) -> float:
    if "rope_theta" in d:
        return float(d["rope_theta"])
    rp = d.get("rope_parameters") or {}
    return float(rp.get("rope_theta", 10000.0))


# -------------------------------------------------------------------- presets
# Public HF architectures used for random-init benches and smoke tests.
_PRESETS: Dict[str, Dict[str, Any]] = {
    "gpt2": dict(model_type="gpt2", n_embd=768, n_layer=12, n_head=12, n_positions=1024, vocab_size=50257),
    "gpt2-medium": dict(model_type="gpt2", n_embd=1024, n_layer=24, n_head=16, n_positions=1024, vocab_size=50257),
    "gpt2-xl": dict(model_type="gpt2", n_embd=1600, n_layer=48, n_head=25, n_positions=1024, vocab_size=50257),
    "gptj-6b": dict(model_type="gptj", n_embd=4096, n_layer=28, n_head=16, n_positions=2048, vocab_size=50400,
                    rotary_dim=64),
    "kogpt-j-350m": dict(model_type="gptj", n_embd=1024, n_layer=20, n_head=16, n_positions=2048,
                         vocab_size=51200, rotary_dim=64),
    "santacoder": dict(model_type="gpt_bigcode", n_embd=2048, n_layer=24, n_head=16, n_positions=2048,
                       vocab_size=49280, multi_query=True),
    "starcoder": dict(model_type="gpt_bigcode", n_embd=6144, n_layer=40, n_head=48, n_positions=8192,
                      vocab_size=49152, multi_query=True),
    "llama2-7b": dict(model_type="llama", hidden_size=4096, num_hidden_layers=32, num_attention_heads=32,
                      num_key_value_heads=32, intermediate_size=11008, vocab_size=32000,
                      max_position_embeddings=4096),
    "llama2-13b": dict(model_type="llama", hidden_size=5120, num_hidden_layers=40, num_attention_heads=40,
                       num_key_value_heads=40, intermediate_size=13824, vocab_size=32000,
                       max_position_embeddings=4096),
    "llama2-70b": dict(model_type="llama", hidden_size=8192, num_hidden_layers=80, num_attention_heads=64,
                       num_key_value_heads=8, intermediate_size=28672, vocab_size=32000,
                       max_position_embeddings=4096),
    # tiny shapes for tests
    "tiny-gpt2": dict(model_type="gpt2", n_embd=64, n_layer=2, n_head=4, n_positions=128, vocab_size=211),
    "tiny-gptj": dict(model_type="gptj", n_embd=64, n_layer=2, n_head=4, n_positions=128, vocab_size=211,
                      rotary_dim=8),
    "tiny-bigcode": dict(model_type="gpt_bigcode", n_embd=64, n_layer=2, n_head=4, n_positions=128,
                         vocab_size=211, multi_query=True),
    "tiny-llama": dict(model_type="llama", hidden_size=64, num_hidden_layers=2, num_attention_heads=4,
                       num_key_value_heads=2, intermediate_size=160, vocab_size=211,
                       max_position_embeddings=128),
    # per-layer design: 3 layers, the last reading layer 0's latent rows; one layer without a feed-forward
    "tiny-timisun": dict(architecture="Timisun", vocab=211, width=48, embedding=dict(scale=4.0), norm=dict(eps=1e-5),
                         layers=[
                             dict(type="latent_attention",
                                  mixer=dict(heads=3, dim=8, vdim=12, kv_rank=24, scale=0.3, mask=dict(size=9)),
                                  mlp=dict(kind="moe", router=dict(experts=5, top=2), expert=dict(ff=20, limit=3.0),
                                           shared=dict(ff=12, limit=1.5))),
                             dict(type="latent_attention",
                                  mixer=dict(heads=2, dim=16, vdim=8, kv_rank=16, scale=0.25), mlp=None),
                             dict(type="latent_attention",
                                  mixer=dict(heads=3, dim=8, vdim=12, kv_rank=24, scale=0.3, mask=dict(size=5),
                                             kv_from=0),
                                  mlp=dict(kind="moe", router=dict(experts=4, top=1), expert=dict(ff=16, limit=2.0))),
                         ]),
    # sequential per-layer design: three residual streams, input convolution, a parallel (attention | delta rule) layer,
    # a decay layer without a feed-forward, grouped heads and partial rotation
    "tiny-babotar": dict(architecture="Babotar", vocab=211, width=48, max_positions=256, norm=dict(eps=1e-5),
                         residual_mult=0.5, streams=3, canon=dict(taps=2),
                         layers=[
                             dict(type="parallel",
                                  mixer=dict(left=dict(heads=4, kv_heads=2, dim=16, vdim=12, scale=0.2, softcap=30.0,
                                                       rot=dict(base=1000.0, dims=8,
                                                                scaling=dict(factor=4.0, original=64, fast=16.0,
                                                                             slow=1.0))),
                                             right=dict(heads=4, kv_heads=2, dim=8, vdim=12, conv=4),
                                             left_scale=0.7, right_scale=1.1),
                                  mlp=dict(kind="dense", ff=64)),
                             dict(type="lightning", mixer=dict(heads=3, dim=8, vdim=16, decay=[0.5, 0.9, 0.99]),
                                  mlp=None),
                         ]),
    # post-norm per-layer design: latent attention with a rotated key part and a gate, differential chunked attention
    # with grouped heads, a layer without a feed-forward, input convolutions, depth averaging, bigram embedding
    "tiny-lamisun": dict(architecture="Lamisun", vocab=211, width=48, norm=dict(eps=1e-5), canon=dict(taps=4),
                         embedding=dict(scale=2.0, bigram=dict(buckets=97, mul_prev=31, mul_cur=7)),
                         layers=[
                             dict(type="attention",
                                  mixer=dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.35, diff=0.2,
                                             mask=dict(size=12)),
                                  mlp=dict(kind="dense", ff=80)),
                             dict(type="latent_attention",
                                  mixer=dict(heads=3, dim=16, rot_dim=8, vdim=12, kv_rank=24, scale=0.2,
                                             rot=dict(base=500.0, dims=8)),
                                  mlp=None),
                             dict(type="latent_attention",
                                  mixer=dict(heads=2, dim=8, rot_dim=4, vdim=16, kv_rank=20, scale=0.3,
                                             rot=dict(base=10000.0, dims=4)),
                                  mlp=dict(kind="dense", ff=64)),
                         ]),
    # sandwich-normed per-layer design: windowed sigmoid attention with pooled blocks, a state-space layer, dense and
    # expert feed-forwards, a looped stretch, token input
    "tiny-fizelix": dict(architecture="Fizelix", vocab=211, width=48, norm=dict(eps=1e-5), embedding=dict(scale=2.0),
                         logit_scale=0.5, token_side=dict(dim=6), loop=dict(start=1, stop=3, times=2),
                         layers=[
                             dict(type="mamba2",
                                  mixer=dict(heads=4, vdim=12, state=8, groups=2, conv=4, norm_groups=2),
                                  mlp=dict(kind="dense", ff=64)),
                             dict(type="attention",
                                  mixer=dict(heads=4, kv_heads=2, dim=8, vdim=12, scale=0.3,
                                             mask=dict(size=7, pool=3), rot=dict(base=1000.0, dims=4)),
                                  mlp=dict(kind="moe", router=dict(experts=5, top=2), expert=dict(ff=20),
                                           shared=dict(ff=12))),
                             dict(type="mamba2",
                                  mixer=dict(heads=3, vdim=16, state=12, groups=1, conv=2, norm_groups=1), mlp=None),
                         ]),
    # TP up to 8 (16 q / kv heads: 2 per rank at TP=8, as Llama-2-7B's 32 give 4)
    "tiny-llama16h": dict(model_type="llama", hidden_size=256, num_hidden_layers=2, num_attention_heads=16,
                          num_key_value_heads=16, intermediate_size=512, vocab_size=211,
                          max_position_embeddings=128),
}


def preset_names():
    return sorted(_PRESETS)


def preset_hf_dict(name: str) -> Dict[str, Any]:
    if name not in _PRESETS:
        raise KeyError(f"unknown preset {name!r}; known: {preset_names()}")
    return dict(_PRESETS[name])


def get_preset(name: str, **overrides) -> ModelConfig:
    cfg = ModelConfig.from_hf_dict(preset_hf_dict(name))
    return replace(cfg, **overrides) if overrides else cfg
