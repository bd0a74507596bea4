"""Decoder whose layers are described one by one (``ModelConfig.layer_specs``) over an fp32 residual stream.

The uniform families run through :class:`~llmss_amd.models.decoder.DecoderLM`; a per-layer design (Timisun, Babotar,
Lamisun, Fizelix) runs through :class:`LayeredLM`, which offers the engine the same surface (``hidden_states`` / ``logits`` over a
:class:`StepInput`, ``allocate_kv_cache``, ``kv_bytes_per_block``, ``plan``) and so shares its scheduler, paged
cache pool, decode graphs and sampler. A layer is either a parallel block (``cfg.parallel_block``)

    h = norm(x) ;  x <- x + (mixer(h) + ffn(h))          x fp32, norm weight stored around zero

or a sequential one over S residual streams x_1 .. x_S (S = 1: the ordinary pre-norm residual), per sublayer

    u = sum_s in[s] x_s ;  y = sublayer(norm(u)) ;  x_t <- sum_s mix[s, t] x_s + c * out[t] * y

where the mixer may read h + causal_conv(h) instead of h; or (``cfg.post_norm``) a sequential block whose norm sits
on each sublayer's output,

    x <- x + norm1(mixer(x + conv1(x))) ;  x <- x + norm2(ffn(x + conv2(x)))

optionally followed by a depth average: what goes on to the next layer is sum_j dwa[j] X_j over the results X_j of
this and all earlier layers (X_0 the embedding); or (``cfg.sandwich``) a sequential block normed on both sides of
each sublayer, its result gated per channel and scaled,

    h = norm_a(x) ;  x <- x + post * rms_norm(sigmoid(W_g h + b) * sublayer(h))          post = norm_b weight * layer scale

optionally followed by a token input (x <- x + rms_norm(W_p (gelu(W_s x) * e)) * w, e the layer's slice of a second
token table); a stretch of such layers may run several times in a row with the same weights (``cfg.loop``), each pass
with cache and state of its own, the embedding added again before every pass but the first. The mixer and the feed-forward are looked up by kind
(``MIXERS`` / ``FFNS``), so another design can combine the same mechanisms with other constants or add its own
beside them. Besides pages of the shared pool a mixer may own per-sequence state (a matrix state per head, the last
inputs of a convolution): ``LayerCache.state`` tensors indexed by the scheduler's state slot of each sequence
(``StepInput.state_slots``); a portion that starts at position 0 starts from an empty state.

Mixer ``parallel`` (ops: linear_f, rope_bias_cache, sink_attn_mix = sink_attn + talk_mix, causal_conv, delta_recurrence,
gated_group_norm): softmax attention with a sink, soft cap, partial scaled rotation and head mixing beside a gated
delta rule, one input GEMM and one output GEMM for both. Mixer ``lightning`` (decay_recurrence, gated_group_norm):
linear attention with a constant decay per head. Feed-forward ``dense`` (glu_act): gated, tanh-form GELU.

Mixer ``latent_attention`` (ops: linear_f, latent_norm_cache, head_absorb, latent_attn, head_expand): the layer
caches one RMS-normed latent row c per token in its paged cache ([blocks, block_size, kv_rank], the step's slots)
and attends with the key projection absorbed into the query: qa_h = W_uk_h^T q_h, p = softmax(scale qa_h . c_j)
over the causal (optionally windowed) keys, out = W_o concat_h(W_uv_h sum_j p_j c_j). A layer with ``kv_from``
projects no latent of its own and reads the named layer's cache with its own W_uk / W_uv. With ``rot_dim`` > 0 every
query head and the cached row carry a rotated part after the latent one (the key's is shared by all heads): the score
is the dot product over the whole row [c | k_rot], the weighted sum reads c alone. ``gate``: the heads' outputs are
multiplied by sigmoid(W_g h) before the output projection.

Mixer ``attention`` (ops: linear_f, qk_norm_cache, sink_attn without a sink, diff_combine): differential attention -
two softmax maps per head over the same values, o = a1 - lambda a2, RMS-normed per head - with RMS-normed queries
and keys and a chunked causal mask. The two maps of a key head are cached as two key heads; the two maps of the query
heads of a group are laid out so that the grouped-query kernel's head mapping serves them (``vshare`` = 2: both key
heads read one value head).

Mixer ``pool_attention`` (ops: linear_f, rope_angles, rope_pairs_cache, pool_update, pool_window_attn): grouped-query
attention without a softmax - a visible key weighs sigmoid(score + bias_h) - over a sliding window and, beyond it,
one mean key / value per block of ``pool`` positions that has wholly left the window; the means live in a pooled cache
beside the pages (one row per block, written when the block's last position is). Mixer ``mamba2`` (causal_conv with
bias, ssd_recurrence, gated_group_norm gate-first): S <- exp(-exp(A) dt) S + dt B x^T, y = S^T C + D x per head.

Feed-forward ``moe`` (ops: moe_router -> fp32 router logits and routing, moe_experts, glu_clamp): sigmoid scores, the
choice made on score + correction, weights = chosen scores normalised; experts and the shared expert use the clamped
gated activation g * sigmoid(1.702 g) * (u + 1); or, by the spec, unnormalised scores that multiply the expert's
INPUT and plain silu(g) * u.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from .. import ops
from ..parallel.dist import TPGroup
from .config import ModelConfig
from .decoder import StepInput
from .weights import ModelWeights, ShardPlan

GLU_ALPHA = 1.702  # the gate's sigmoid slope of the clamped gated activation


class LatentAttention:
    """Mixer ``latent_attention``."""

    @staticmethod
    def cache_row(spec) -> Optional[int]:
        """Numbers cached per token by a layer of this kind (None: it reads another layer's cache)."""
        return spec.kv_rank + spec.rot_dim if spec.kv_from is None else None

    @staticmethod
    def forward(model: "LayeredLM", i: int, W, spec, h, inp: StepInput, cu, caches):
        dt = model.dtype
        H, dim, R, rot = spec.heads, spec.dim, spec.kv_rank, spec.rot_dim
        qc = ops.linear_f(h, W.qc, dt)  # [T, H * (dim + rot) (+ R + rot) (+ H * vdim)]: queries, raw latent, gate
        cache = caches[i if spec.kv_from is None else spec.kv_from][0]
        qa = ops.head_absorb(qc, W.uk_t, ops.latent_qa_dtype(cache), extra=rot)
        if W.own_kv:
            cs = model.angles(inp, W.rot_key, W.freqs) if rot else None
            ops.latent_norm_cache(qc, H * (dim + rot), R, W.kv_norm, model.cfg.norm_eps, cache, inp.slots, rot, cs,
                                  qa if rot else None, 0, dim)
        nd = inp.num_decode if inp.kind == "extend" else 0
        if nd and nd < qa.shape[0]:
            # mixed step: the single-token rows take the decode form of the kernel (their keys split over
            # workgroups), the portions the prompt form - as DecoderLM sends its decode rows to the decode kernel
            o = torch.cat([
                ops.latent_attn(qa[:nd], cache, inp.block_tables[:nd], model.decode_cu(nd, qa.device),
                                inp.ctx_lens[:nd], spec.window, spec.scale, max_qlen=1, max_ctx=inp.max_ctx),
                ops.latent_attn(qa[nd:], cache, inp.block_tables[nd:], inp.cu_seqlens, inp.ctx_lens[nd:],
                                spec.window, spec.scale, max_qlen=max(1, inp.max_seqlen))])
        else:
            single = inp.kind == "decode" or (nd and nd == qa.shape[0])
            o = ops.latent_attn(qa, cache, inp.block_tables, cu, inp.ctx_lens, spec.window, spec.scale,
                                max_qlen=1 if single else max(1, inp.max_seqlen),
                                max_ctx=inp.max_ctx if single else 0)
        y = ops.head_expand(o, W.uv, dt)
        if W.gate_col is not None:
            y = ops.gate_mul(y, qc, W.gate_col)
        return ops.linear_f(y, W.o, dt)


class DiffAttention:
    """Mixer ``attention``: differential softmax attention over paged key / value rows."""

    @staticmethod
    def cache_row(spec) -> Optional[int]:
        return spec.kv_heads * (2 * spec.dim + spec.vdim)

    @staticmethod
    def allocate(model: "LayeredLM", spec, num_blocks: int, block_size: int, num_slots: int):
        dt, dev = model.dtype, model.device
        return (torch.zeros(num_blocks, block_size, spec.kv_heads * 2 * spec.dim, dtype=dt, device=dev),
                torch.zeros(num_blocks, block_size, spec.kv_heads * spec.vdim, dtype=dt, device=dev), {})

    @staticmethod
    def forward(model: "LayeredLM", i: int, W, spec, h, inp: StepInput, cu, caches):
        dt, eps, c = model.dtype, model.cfg.norm_eps, W.cols
        kc, vc = caches[i][0], caches[i][1]
        H, G = spec.heads, spec.kv_heads
        proj = ops.linear_f(h, W.proj, dt)
        q = ops.qk_norm_cache(proj, c["q"], c["k"], c["v"], W.q_norm, W.k_norm, eps, kc, vc, inp.slots, H, G, 2,
                              spec.dim, spec.vdim)
        single = inp.kind == "decode"
        # the two maps as 2 H query heads on 2 G key heads; both key heads of a pair read one value head
        O = ops.sink_attn(q, kc, vc, inp.block_tables, cu, inp.ctx_lens, 2 * H, 2 * G, spec.dim, spec.vdim, spec.scale,
                          0.0, False, max_qlen=1 if single else max(1, inp.max_seqlen),
                          num_decode=0 if single else inp.num_decode, sink=False, chunk=spec.chunk, vshare=2,
                          precise=True)
        y = ops.diff_combine(O, W.lam, eps, 1.0 - spec.diff, H, G, spec.vdim, dt)
        return ops.linear_f(y, W.o, dt)


class MoEFeedForward:
    """Feed-forward ``moe``."""

    @staticmethod
    def forward(model: "LayeredLM", W, spec, h):
        dt = model.dtype
        idx, wts = ops.moe_router(h, W.router, W.correction, spec.top, spec.normalize)
        sh = None
        if W.shared_gu is not None:
            # (a sandwich block's gate logits ride in this GEMM as extra columns: model.proj)
            gu = model.proj = ops.linear_f(h, W.shared_gu, dt)
            if spec.shared is not None:
                a = ops.glu_act(gu, spec.shared.ff, "silu") if spec.act == "silu" else \
                    ops.glu_clamp(gu, spec.shared.ff, spec.shared.limit, GLU_ALPHA)
                sh = ops.linear_f(a, W.shared_down, dt)
        # combine=False: on the GPU the weighted sum over the chosen experts happens inside the next residual add
        return ops.moe_experts(h, idx, wts, W.gate, W.up, W.down, spec.expert.limit, GLU_ALPHA, shared=sh,
                               combine=False, act=spec.act, weight_input=spec.weight_input)


class ParallelMixer:
    """Mixer ``parallel``: sink attention (paged k / v rows) beside a gated delta rule (matrix state and convolution
    tail per sequence)."""

    @staticmethod
    def cache_row(spec) -> Optional[int]:
        return spec.left.kv_heads * (spec.left.dim + spec.left.vdim)

    @staticmethod
    def allocate(model: "LayeredLM", spec, num_blocks: int, block_size: int, num_slots: int):
        a, r = spec.left, spec.right
        dt, dev = model.dtype, model.device
        C = 2 * r.kv_heads * r.dim + r.heads * r.vdim
        return (torch.zeros(num_blocks, block_size, a.kv_heads * a.dim, dtype=dt, device=dev),
                torch.zeros(num_blocks, block_size, a.kv_heads * a.vdim, dtype=dt, device=dev),
                {"S": torch.zeros(num_slots, r.heads, r.dim, r.vdim, dtype=torch.float32, device=dev),
                 "tail": torch.zeros(num_slots, max(r.conv - 1, 0), C, dtype=torch.float32, device=dev)})

    @staticmethod
    def state_bytes(spec) -> int:
        r = spec.right
        return 4 * (r.heads * r.dim * r.vdim + max(r.conv - 1, 0) * (2 * r.kv_heads * r.dim + r.heads * r.vdim))

    @staticmethod
    def forward(model: "LayeredLM", i: int, W, spec, h, inp: StepInput, cu, caches):
        dt, eps = model.dtype, model.cfg.norm_eps
        a, r, c = spec.left, spec.right, W.cols
        kc, vc, st = caches[i]
        T = h.shape[0]
        proj = ops.linear_f(h, W.proj, dt)
        # left: softmax attention with a sink over the paged cache, the heads' weights mixed afterwards
        q = ops.rope_bias_cache(proj, c["lq"], c["lk"], c["lv"], W.bias, inp.positions, W.angles,
                                a.rot.dims if a.rot is not None else 0, kc, vc, inp.slots, a.heads, a.kv_heads, a.dim,
                                a.vdim)
        single = inp.kind == "decode"
        nl, nr = a.heads * a.vdim, r.heads * r.vdim
        both = torch.empty(T, nl + nr, dtype=dt, device=h.device)  # [left | right] rows for the one output GEMM
        ops.sink_attn_mix(q, kc, vc, inp.block_tables, cu, inp.ctx_lens, W.talk, spec.left_scale, a.heads, a.kv_heads,
                          a.dim, a.vdim, a.scale, a.softcap, both[:, :nl],
                          max_qlen=1 if single else max(1, inp.max_seqlen), num_decode=0 if single else inp.num_decode,
                          max_ctx=inp.max_ctx)
        # right: short convolution + SiLU on q | k | v, then the gated delta rule over the sequence's matrix state
        nqk = r.kv_heads * r.dim
        qkv = ops.causal_conv(proj[:, c["rq"]:c["rq"] + 2 * nqk + nr], W.conv, st["tail"], cu, inp.ctx_lens,
                              inp.state_slots, False, True, torch.float32)
        o = ops.delta_recurrence(qkv[:, :nqk], qkv[:, nqk:2 * nqk], qkv[:, 2 * nqk:], proj[:, c["ra"]:c["ra"] + r.heads],
                                 proj[:, c["rb"]:c["rb"] + r.heads], W.A_log, W.dt_bias, st["S"], cu, inp.ctx_lens,
                                 inp.state_slots, r.heads, r.kv_heads, r.dim, r.vdim)
        ops.gated_group_norm(o, proj[:, c["rg"]:c["rg"] + nr], W.norm, eps, "silu", spec.right_scale,
                             out=both[:, nl:])
        return ops.linear_f(both, W.o, dt)


class DecayMixer:
    """Mixer ``lightning``: S <- decay_h S + k v^T, o = S^T q per head, then a gated RMS norm over all heads."""

    @staticmethod
    def cache_row(spec) -> Optional[int]:
        return None

    @staticmethod
    def allocate(model: "LayeredLM", spec, num_blocks: int, block_size: int, num_slots: int):
        return (None, None, {"S": torch.zeros(num_slots, spec.heads, spec.dim, spec.vdim, dtype=torch.float32,
                                              device=model.device)})

    @staticmethod
    def state_bytes(spec) -> int:
        return 4 * spec.heads * spec.dim * spec.vdim

    @staticmethod
    def forward(model: "LayeredLM", i: int, W, spec, h, inp: StepInput, cu, caches):
        dt, c = model.dtype, W.cols
        nqk, nv = spec.heads * spec.dim, spec.heads * spec.vdim
        proj = ops.linear_f(h, W.proj, dt)
        o = ops.decay_recurrence(proj[:, c["q"]:c["q"] + nqk], proj[:, c["k"]:c["k"] + nqk],
                                 proj[:, c["v"]:c["v"] + nv], W.decay, caches[i][2]["S"], cu, inp.ctx_lens,
                                 inp.state_slots, spec.heads, spec.dim, spec.vdim, True)
        y = ops.gated_group_norm(o, proj[:, c["g"]:c["g"] + nv], W.norm, model.cfg.norm_eps, "sigmoid", 1.0,
                                 out_dtype=dt)
        return ops.linear_f(y, W.o, dt)


class DenseFeedForward:
    """Feed-forward ``dense``: down(act(gate h) * (up h)), gate and up as one GEMM; ungated: down(act(up h))."""

    @staticmethod
    def forward(model: "LayeredLM", W, spec, h):
        dt = model.dtype
        if not spec.gated:
            return ops.linear_f(ops.act_fn(ops.linear_f(h, W.gu, dt), spec.act, W.act_params), W.down, dt)
        gu = model.proj = ops.linear_f(h, W.gu, dt)  # (columns past 2 ff: a sandwich block's gate logits)
        return ops.linear_f(ops.glu_act(gu, spec.ff, spec.act), W.down, dt)


class PoolAttention:
    """Mixer ``pool_attention``: sigmoid-weighted grouped-query attention over a sliding window of the paged key /
    value rows plus one mean row per block of ``pool`` positions behind the window."""

    @staticmethod
    def cache_row(spec) -> Optional[int]:
        return spec.kv_heads * (spec.dim + spec.vdim)

    @staticmethod
    def pooled_per_page(spec, block_size: int) -> int:
        return -(-block_size // spec.pool) if spec.pool else 0

    @staticmethod
    def allocate(model: "LayeredLM", spec, num_blocks: int, block_size: int, num_slots: int):
        dt, dev = model.dtype, model.device
        per = PoolAttention.pooled_per_page(spec, block_size)
        pooled = {}
        if per:  # the blocks' means: row (page of the block's first position, rank among the blocks starting there)
            pooled = {"kp": torch.zeros(num_blocks, per, spec.kv_heads * spec.dim, dtype=dt, device=dev),
                      "vp": torch.zeros(num_blocks, per, spec.kv_heads * spec.vdim, dtype=dt, device=dev)}
        return (torch.zeros(num_blocks, block_size, spec.kv_heads * spec.dim, dtype=dt, device=dev),
                torch.zeros(num_blocks, block_size, spec.kv_heads * spec.vdim, dtype=dt, device=dev), pooled)

    @staticmethod
    def extra_bytes_per_block(spec, block_size: int, elem: int) -> int:
        return elem * PoolAttention.pooled_per_page(spec, block_size) * spec.kv_heads * (spec.dim + spec.vdim)

    @staticmethod
    def forward(model: "LayeredLM", i: int, W, spec, h, inp: StepInput, cu, caches):
        dt, c = model.dtype, W.cols
        kc, vc, pooled = caches[i]
        proj = model.proj = ops.linear_f(h, W.proj, dt)
        cs = model.angles(inp, W.rot_key, W.freqs) if W.freqs is not None else None
        q = ops.rope_pairs_cache(proj, c["q"], c["k"], c["v"], cs, kc, vc, inp.slots, spec.heads, spec.kv_heads,
                                 spec.dim, spec.vdim)
        kp, vp = pooled.get("kp"), pooled.get("vp")
        single = inp.kind == "decode"
        if spec.pool:
            ops.pool_update(kc, vc, kp, vp, inp.block_tables, cu, inp.ctx_lens, spec.pool,
                            max_qlen=1 if single else max(1, inp.max_seqlen))
        y = ops.pool_window_attn(q, kc, vc, kp, vp, inp.block_tables, cu, inp.ctx_lens, W.pb, spec.heads,
                                 spec.kv_heads, spec.dim, spec.vdim, spec.scale, spec.window, spec.pool, dt,
                                 max_qlen=1 if single else max(1, inp.max_seqlen),
                                 num_decode=0 if single else inp.num_decode, max_ctx=inp.max_ctx)
        return ops.linear_f(y, W.o, dt)


class SSDMixer:
    """Mixer ``mamba2``: x | B | C through a short causal convolution with bias and SiLU, the scalar-decay state-space
    recurrence over a matrix state per head, the result gated by silu(z) and then normed in groups."""

    @staticmethod
    def cache_row(spec) -> Optional[int]:
        return None

    @staticmethod
    def allocate(model: "LayeredLM", spec, num_blocks: int, block_size: int, num_slots: int):
        dev = model.device
        return (None, None,
                {"S": torch.zeros(num_slots, spec.heads, spec.state, spec.vdim, dtype=torch.float32, device=dev),
                 "tail": torch.zeros(num_slots, max(spec.conv - 1, 0), spec.conv_channels, dtype=torch.float32,
                                     device=dev)})

    @staticmethod
    def state_bytes(spec) -> int:
        return 4 * (spec.heads * spec.state * spec.vdim + max(spec.conv - 1, 0) * spec.conv_channels)

    @staticmethod
    def forward(model: "LayeredLM", i: int, W, spec, h, inp: StepInput, cu, caches):
        dt, c = model.dtype, W.cols
        st = caches[i][2]
        inner, gn = spec.inner, spec.groups * spec.state
        proj = model.proj = ops.linear_f(h, W.proj, dt)
        xbc = ops.causal_conv(proj[:, c["xbc"]:c["xbc"] + spec.conv_channels], W.conv, st["tail"], cu, inp.ctx_lens,
                              inp.state_slots, False, True, dt, bias=W.conv_b)
        y = ops.ssd_recurrence(xbc[:, :inner], xbc[:, inner:inner + gn], xbc[:, inner + gn:],
                               proj[:, c["dt"]:c["dt"] + spec.heads], W.A_log, W.dt_bias, W.D, st["S"], cu,
                               inp.ctx_lens, inp.state_slots, spec.heads, spec.groups, spec.state, spec.vdim)
        y = ops.gated_group_norm(y, proj[:, c["z"]:c["z"] + inner], W.norm, model.cfg.norm_eps, "silu", 1.0,
                                 out_dtype=dt, groups=spec.norm_groups, gate_first=True)
        return ops.linear_f(y, W.o, dt)


MIXERS = {"latent_attention": LatentAttention, "parallel": ParallelMixer, "lightning": DecayMixer,
          "attention": DiffAttention, "pool_attention": PoolAttention, "mamba2": SSDMixer}
FFNS = {"moe": MoEFeedForward, "dense": DenseFeedForward}


class LayeredLM:
    def __init__(self, cfg: ModelConfig, weights: ModelWeights, tp: Optional[TPGroup] = None):
        if not cfg.layer_specs:
            raise ValueError("LayeredLM needs a config with layer_specs")
        self.cfg = cfg
        self.w = weights
        self.tp = tp or TPGroup()
        if self.tp.size != 1:
            raise NotImplementedError(f"{cfg.model_type}: tensor parallelism is not implemented for per-layer designs")
        for s in cfg.layer_specs:
            if s.mixer.kind not in MIXERS:
                raise ValueError(f"unknown mixer kind {s.mixer.kind!r}")
            if s.mlp is not None and s.mlp.kind not in FFNS:
                raise ValueError(f"unknown feed-forward kind {s.mlp.kind!r}")
        self.plan = ShardPlan(1, 0, cfg.num_heads, 0, 1, cfg.intermediate_size, weights.head.w.shape[0])
        # what the engine asks of every model: no TP decode schedules, no fp8 cache rows here
        self.kv_fp8 = False
        self.tbo_min = 0
        self.rsag_mode = self.col_mode = "0"
        self.rsag: set = set()
        self.col: set = set()
        self.col_chunks = 0
        self.overlap_rows = None
        self.bucket_bytes = 0
        self.gqa_mfma: set = set()
        self._cu_decode = {}
        self._angles = {}
        self.tap = None  # tap(i, x): called with the fp32 residual after layer (run) i (debugging, tests)
        self.proj = None  # the last sublayer's first GEMM output (a sandwich block reads its gate logits there)

    @property
    def device(self):
        return self.w.wte.device

    @property
    def dtype(self):
        return self.w.wte.dtype

    def overlap_split(self, B: int) -> int:
        return 0

    def gemm_shapes(self):
        """The dense projections that run on the autotuned MFMA GEMM (ops.linear_f -> ops/hip.py linear), one entry
        per distinct [N, K]: query | latent, output, the shared expert's two products and the head. The engine's
        autotuner times plans for them per decode bucket (ops/autotune.py)."""
        from ..ops.autotune import GemmShape

        if self.dtype != torch.bfloat16:
            return {}
        out = {}

        def put(name, w):
            N, K = w.shape
            if K % 16 == 0 and N % 8 == 0 and (N, K) not in {(s.N, s.K) for s in out.values()}:
                out[f"{name}_{N}x{K}"] = GemmShape(N, K)
        for L in self.w.layers:
            for nm in ("qc", "proj", "o"):
                if hasattr(L.mix, nm):
                    put(nm, getattr(L.mix, nm))
            for nm in ("shared_gu", "shared_down", "gu", "down"):
                if getattr(L, "mlp", None) is not None and getattr(L.mlp, nm, None) is not None and \
                        getattr(L.mlp, nm).dim() == 2:
                    put(nm, getattr(L.mlp, nm))
        put("head", self.w.head.w)
        return out

    # --------------------------------------------------------------------------------- cache
    def _run_specs(self):
        """The spec of every layer RUN (a looped stretch repeats): caches and state are per run."""
        return [self.cfg.layer_specs[i] for i in self.cfg.layer_runs()]

    def _cache_rows(self) -> List[Optional[int]]:
        return [MIXERS[s.mixer.kind].cache_row(s.mixer) for s in self._run_specs()]

    def kv_bytes_per_block(self, block_size: int) -> int:
        n = sum(block_size * r * self.w.wte.element_size() for r in self._cache_rows() if r)
        n += sum(MIXERS[s.mixer.kind].extra_bytes_per_block(s.mixer, block_size, self.w.wte.element_size())
                 for s in self._run_specs()
                 if hasattr(MIXERS[s.mixer.kind], "extra_bytes_per_block"))
        return max(1, n)

    @property
    def needs_state(self) -> bool:
        """Some mixer keeps per-sequence state besides its pages: steps must carry the sequences' state slots."""
        return any(hasattr(MIXERS[s.mixer.kind], "state_bytes") for s in self.cfg.layer_specs) or \
            bool(self.cfg.canon_taps > 1) or self.cfg.bigram is not None

    def _canon_sublayers(self) -> int:
        return 2 if self.cfg.canon_ffn else 1

    def state_bytes_per_slot(self) -> int:
        n = sum(MIXERS[s.mixer.kind].state_bytes(s.mixer) for s in self._run_specs()
                if hasattr(MIXERS[s.mixer.kind], "state_bytes"))
        n += 8 if self.cfg.bigram is not None else 0
        return n + 4 * max(self.cfg.canon_taps - 1, 0) * self.cfg.hidden_size * len(self.cfg.layer_specs) * \
            self._canon_sublayers()

    def allocate_kv_cache(self, num_blocks: int, block_size: int, num_slots: int = 0):
        """One entry per layer run (a looped stretch of layers has an entry per pass). Latent attention: (rows, None), a layer that reads another layer's rows holding that
        layer's pair. Mixers with an ``allocate`` of their own: (key pages, value pages, {name: per-slot state});
        ``num_slots`` state slots, one per running sequence. The input convolution's tails of all layers live in
        ``self.canon_tail`` [layers (x 2 when the feed-forward has a convolution too: mixer, feed-forward), slots,
        taps - 1, W], the token before each sequence's next one (bigram embedding) in ``self.prev_token`` [slots]."""
        caches: list = []
        for s, r in zip(self._run_specs(), self._cache_rows()):
            mx = MIXERS[s.mixer.kind]
            if hasattr(mx, "allocate"):
                if num_slots <= 0 and hasattr(mx, "state_bytes"):
                    raise ValueError(f"{self.cfg.model_type}: the cache needs state slots (num_slots)")
                caches.append(mx.allocate(self, s.mixer, num_blocks, block_size, num_slots))
            elif r:
                caches.append((torch.zeros(num_blocks, block_size, r, dtype=self.dtype, device=self.device), None))
            else:
                caches.append(caches[s.mixer.kv_from])
        if self.cfg.canon_taps > 1:
            self.canon_tail = torch.zeros(len(caches) * self._canon_sublayers(), max(num_slots, 1),
                                          self.cfg.canon_taps - 1, self.cfg.hidden_size, dtype=torch.float32,
                                          device=self.device)
        if self.cfg.bigram is not None:
            self.prev_token = torch.zeros(max(num_slots, 1), dtype=torch.int64, device=self.device)
        return caches

    # ---------------------------------------------------------------------------- forward
    def decode_cu(self, B: int, device) -> torch.Tensor:
        cu = self._cu_decode.get((B, str(device)))
        if cu is None:
            cu = self._cu_decode[(B, str(device))] = torch.arange(B + 1, dtype=torch.int32, device=device)
        return cu

    def _cu(self, inp: StepInput) -> torch.Tensor:
        """Row boundaries of every sequence of the step, single-token rows first (the order of block_tables)."""
        dev = inp.input_ids.device
        if inp.kind == "decode":
            return self.decode_cu(inp.input_ids.shape[0], dev)
        if inp.num_decode:
            return torch.cat([torch.arange(inp.num_decode, dtype=torch.int32, device=dev),
                              inp.cu_seqlens.to(torch.int32) + inp.num_decode])
        return inp.cu_seqlens

    def hidden_states(self, inp: StepInput, kv_caches) -> torch.Tensor:
        if inp.block_tables is None or inp.ctx_lens is None or not any(t is not None for t in kv_caches[0]):
            raise ValueError(f"{self.cfg.model_type} attends through its paged cache: the step needs block tables, "
                             f"context lengths and a cache (a cache-less recompute step is not supported)")
        if self.cfg.sandwich:
            return self._sandwich_blocks(inp, kv_caches)
        if self.cfg.post_norm:
            return self._postnorm_blocks(inp, kv_caches)
        if not self.cfg.parallel_block:
            return self._sequential_blocks(inp, kv_caches)
        cfg, w = self.cfg, self.w
        eps, off, dt = cfg.norm_eps, cfg.norm_offset, self.dtype
        cu = self._cu(inp)
        x = ops.embed_scaled(inp.input_ids, w.wte, cfg.embedding_scale)
        a = f = None
        for i, (L, spec) in enumerate(zip(w.layers, cfg.layer_specs)):
            h = ops.resid_add_norm(x, a, f, L.norm1, off, eps, dt)
            if self.tap is not None and i:
                self.tap(i - 1, x)
            a = MIXERS[spec.mixer.kind].forward(self, i, L.mix, spec.mixer, h, inp, cu, kv_caches)
            f = FFNS[spec.mlp.kind].forward(self, L.mlp, spec.mlp, h) if spec.mlp is not None else None
        h = ops.resid_add_norm(x, a, f, w.lnf_w, off, eps, dt)
        if self.tap is not None:
            self.tap(len(w.layers) - 1, x)
        return h

    def _sequential_blocks(self, inp: StepInput, kv_caches) -> torch.Tensor:
        """Sequential blocks over the residual streams. The write-back of one sublayer and the read + norm of the
        next are one op (stream_add_norm), as the residual add and the next norm are for the other families."""
        cfg, w, dt = self.cfg, self.w, self.dtype
        if self.needs_state and inp.state_slots is None:
            raise ValueError(f"{cfg.model_type} keeps per-sequence state: the step needs the sequences' state slots")
        eps, c, rms = cfg.norm_eps, cfg.residual_mult, cfg.norm == "rmsnorm"
        cu = self._cu(inp)
        x = ops.embed_streams(inp.input_ids, inp.positions, w.wte, w.wpe, max(cfg.streams, 1))
        y = prev = None  # the sublayer output not yet written back, and its stream weights
        for i, (L, spec) in enumerate(zip(w.layers, cfg.layer_specs)):
            canon = L.canon is not None
            h = ops.stream_add_norm(x, y, prev.mix if prev else None, prev.outw if prev else None, c, L.hc1.inw,
                                    L.norm1, eps, rms, torch.float32 if canon else dt)
            if self.tap is not None and i:
                self.tap(i - 1, x.sum(0))
            if canon:
                tail = self.canon_tail[i] if cfg.canon_taps > 1 else None
                h = ops.causal_conv(h, L.canon, tail, cu, inp.ctx_lens, inp.state_slots, True, False, dt)
            y, prev = MIXERS[spec.mixer.kind].forward(self, i, L.mix, spec.mixer, h, inp, cu, kv_caches), L.hc1
            if spec.mlp is not None:
                h = ops.stream_add_norm(x, y, prev.mix, prev.outw, c, L.hc2.inw, L.norm2, eps, rms, dt)
                y, prev = FFNS[spec.mlp.kind].forward(self, L.mlp, spec.mlp, h), L.hc2
        h = ops.stream_add_norm(x, y, prev.mix, prev.outw, c, None, w.lnf_w, eps, rms, dt)
        if self.tap is not None:
            self.tap(len(w.layers) - 1, x.sum(0))
        return h

    def angles(self, inp: StepInput, key: tuple, freqs: torch.Tensor) -> torch.Tensor:
        """(cos, sin) [T, len(freqs), 2] of the step's positions, formed once per step and distinct rotation ``key``."""
        cs = self._angles.get(key)
        if cs is None:
            cs = self._angles[key] = ops.rope_angles(inp.positions, freqs)
        return cs

    def _postnorm_blocks(self, inp: StepInput, kv_caches) -> torch.Tensor:
        """Blocks normed on the sublayers' outputs, with input convolutions and the depth average. ``hist`` [L + 2,
        T, W] fp32 holds the layers' results: layer i works in place on hist[i + 1], which the step before filled
        with the layer's input - the embedding for layer 0, the depth average leaving layer i - 1 afterwards (without
        depth averaging the one row block is carried along)."""
        cfg, w, dt = self.cfg, self.w, self.dtype
        if self.needs_state and inp.state_slots is None:
            raise ValueError(f"{cfg.model_type} keeps per-sequence state: the step needs the sequences' state slots")
        eps = cfg.norm_eps
        cu = self._cu(inp)
        T, L = inp.input_ids.shape[0], len(w.layers)
        self._angles = {}
        dwa = cfg.depth_average
        hist = torch.empty(L + 2 if dwa else 2, T, cfg.hidden_size, dtype=torch.float32, device=self.device)
        if cfg.bigram is not None:
            ops.embed_bigram(inp.input_ids, inp.positions, w.wte, cfg.embedding_scale, w.extra["bigram"],
                             cfg.bigram.mul_prev, cfg.bigram.mul_cur, self.prev_token, cu, inp.ctx_lens,
                             inp.state_slots, hist)
        else:
            hist[0].copy_(ops.embed_scaled(inp.input_ids, w.wte, cfg.embedding_scale))
            hist[1].copy_(hist[0])
        nsub = self._canon_sublayers()
        x = hist[1]
        for i, (Lw, spec) in enumerate(zip(w.layers, cfg.layer_specs)):
            n = i + 1 if dwa else 1

            def read(canon, k):  # what a sublayer reads: x + conv(x), or x, in the storage type
                if canon is None:
                    return x.to(dt)
                tail = self.canon_tail[nsub * i + k] if cfg.canon_taps > 1 else None
                return ops.causal_conv(x, canon, tail, cu, inp.ctx_lens, inp.state_slots, True, False, dt)
            y = MIXERS[spec.mixer.kind].forward(self, i, Lw.mix, spec.mixer, read(Lw.canon1, 0), inp, cu, kv_caches)
            last = spec.mlp is None
            x = ops.resid_norm_add(hist, n, y, Lw.norm1, eps, Lw.dwa if last and dwa else None)
            if not last:
                y = FFNS[spec.mlp.kind].forward(self, Lw.mlp, spec.mlp, read(Lw.canon2, 1))
                x = ops.resid_norm_add(hist, n, y, Lw.norm2, eps, Lw.dwa if dwa else None)
            if self.tap is not None:
                self.tap(i, x)
        self._angles = {}
        return ops.resid_add_norm(x, None, None, w.lnf_w, 0.0, eps, dt)

    def _sandwich_blocks(self, inp: StepInput, kv_caches) -> torch.Tensor:
        """Blocks normed on both sides of their sublayers. Every sublayer's closing op (the gated, normed, scaled
        residual add, or the token input after it) also forms what the next reader takes - the next sublayer's normed
        input, with the embedding added first where a new pass of a looped stretch begins - as the residual add and
        the next norm are one op for the other families. The gate logits come out of the sublayer's own first GEMM
        (``self.proj``). With a ``tap`` the closing ops run unfused, so that the tap sees the residual as the layer
        leaves it."""
        cfg, w, dt = self.cfg, self.w, self.dtype
        if self.needs_state and inp.state_slots is None:
            raise ValueError(f"{cfg.model_type} keeps per-sequence state: the step needs the sequences' state slots")
        eps = cfg.norm_eps
        cu = self._cu(inp)
        self._angles = {}
        runs = cfg.layer_runs()
        x = ops.embed_scaled(inp.input_ids, w.wte, cfg.embedding_scale)
        x0 = x.clone() if cfg.loop else None
        W_ = cfg.hidden_size
        h = ops.sandwich_add_norm(x, None, None, None, None, eps, None, w.layers[runs[0]].norm1, dt)
        for r, i in enumerate(runs):
            L, spec = w.layers[i], cfg.layer_specs[i]
            last = r + 1 == len(runs)
            nxt = w.lnf_w if last else w.layers[runs[r + 1]].norm1
            # the embedding comes back in before a pass of the looped stretch other than the first
            add = x0 if not last and cfg.loop and runs[r + 1] == cfg.loop[0] and r + 1 > cfg.loop[0] else None
            if self.tap is not None:
                tail = (None, None)  # close the layer first, tap, then add / norm on their own
            else:
                tail = (add, nxt)
            side = L.side_gate is not None
            y = MIXERS[spec.mixer.kind].forward(self, r, L.mix, spec.mixer, h, inp, cu, kv_caches)
            c0 = L.mix.cols["rg"]
            after = (None, L.norm2) if spec.mlp is not None else ((None, None) if side else tail)
            h = ops.sandwich_add_norm(x, y, self.proj[:, c0:c0 + W_], L.rg1_b, L.post1, eps, *after, dt)
            if spec.mlp is not None:
                y = FFNS[spec.mlp.kind].forward(self, L.mlp, spec.mlp, h)
                after = (None, None) if side else tail
                h = ops.sandwich_add_norm(x, y, self.proj[:, L.rg2_col:L.rg2_col + W_], L.rg2_b, L.post2, eps, *after,
                                          dt)
            if side:
                h = ops.token_side_add(x, inp.input_ids, w.extra["side"], L.side_col, L.side_gate, L.side_proj,
                                       L.side_norm, eps, *tail, dt)
            if self.tap is not None:
                self.tap(r, x)
                h = ops.sandwich_add_norm(x, None, None, None, None, eps, add, nxt, dt)
        self._angles = {}
        self.proj = None
        return h

    @property
    def vocab_lo(self) -> int:
        return 0

    def local_logits(self, h: torch.Tensor) -> torch.Tensor:
        return ops.linear_f(h, self.w.head.w, self.dtype)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        """[B, H] -> [B, V padded to 16] against the embedding table itself (no embedding scale)."""
        return self.local_logits(h)

    def forward(self, inp: StepInput, kv_caches) -> torch.Tensor:
        h = self.hidden_states(inp, kv_caches)
        if inp.last_idx is not None:
            h = h.index_select(0, inp.last_idx)
        return self.logits(h)

    __call__ = forward


def create_model(cfg: ModelConfig, weights: ModelWeights, tp: Optional[TPGroup] = None):
    """The model class of a config: per-layer designs -> LayeredLM, the uniform families -> DecoderLM."""
    if cfg.layer_specs:
        return LayeredLM(cfg, weights, tp)
    from .decoder import DecoderLM

    return DecoderLM(cfg, weights, tp)
