"""Plain-PyTorch definitions of every op (CPU execution path and the numerics oracle).

Each function has exactly the semantics of its gfx950 HIP kernel in ``llmss_amd/csrc`` and is
used (a) when the tensors live on the CPU (the TP=1 CPU plumbing configuration, gloo
multi-process tests) and (b) by the GPU tests as the fp32 reference. There is no runtime switch
from a GPU tensor to these functions: ``llmss_amd.ops`` routes by device only.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import numpy as np
import torch
import torch.nn.functional as F

ACTS = {"none": 0, "gelu_tanh": 1, "gelu": 2, "relu": 3, "silu_glu": 4}


def _act(x: torch.Tensor, act: str) -> torch.Tensor:
    if act in (None, "none"):
        return x
    if act == "gelu_tanh":
        return F.gelu(x, approximate="tanh")
    if act == "gelu":
        return F.gelu(x)
    if act == "relu":
        return F.relu(x)
    raise ValueError(act)


def add_norm(x, weight, bias, eps: float, rms: bool, residual: Optional[torch.Tensor] = None,
             ) -> Tuple[torch.Tensor, torch.Tensor]:
    """r = x (+ residual) [rounded to x.dtype]; y = norm(r) * w (+ b). Returns (y, r)."""
    r = x if residual is None else (x.float() + residual.float()).to(x.dtype)
    rf = r.float()
    if rms:
        y = rf * torch.rsqrt(rf.pow(2).mean(-1, keepdim=True) + eps)
    else:
        mu = rf.mean(-1, keepdim=True)
        var = (rf - mu).pow(2).mean(-1, keepdim=True)
        y = (rf - mu) * torch.rsqrt(var + eps)
    y = y * weight.float()
    if bias is not None:
        y = y + bias.float()
    return y.to(x.dtype), r


def embed(ids: torch.Tensor, wte: torch.Tensor, positions: Optional[torch.Tensor] = None,
          wpe: Optional[torch.Tensor] = None) -> torch.Tensor:
    ids = ids.clamp(0, wte.shape[0] - 1)
    out = wte[ids]
    if wpe is not None:
        out = (out.float() + wpe[positions].float()).to(wte.dtype)
    return out


def rope_tables(max_pos: int, rot: int, theta: float, device=None):
    inv = 1.0 / (theta ** (torch.arange(0, rot, 2, dtype=torch.float64) / rot))
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None, :]
    return ang.cos().float().to(device), ang.sin().float().to(device)


def rope_interleave_perm(D: int, rot: int) -> torch.Tensor:
    """Head-dim order that turns neox RoPE (pairs (j, j + rot/2)) into adjacent pairs (2j, 2j + 1): new
    dim 2j <- old j, 2j + 1 <- old j + rot/2, dims >= rot unchanged. Applied to the q and k rows of the
    fused QKV weight at load, attention scores are unchanged (q and k permute alike, V does not) and the
    rotation becomes the gptj form, which the QKV GEMM epilogue applies in-register for any tile width."""
    h = rot // 2
    first = torch.stack([torch.arange(h), torch.arange(h) + h], 1).reshape(-1)
    return torch.cat([first, torch.arange(rot, D)])


def rope_interleave_rows(t: torch.Tensor, nh: int, nkv: int, D: int, rot: int) -> torch.Tensor:
    """Permute the q and k head rows of a fused [(nh + 2 nkv) * D, ...] QKV weight / bias (see
    rope_interleave_perm); v rows stay."""
    perm = rope_interleave_perm(D, rot).to(t.device)
    nqk = (nh + nkv) * D
    idx = (torch.arange(nh + nkv, device=t.device)[:, None] * D + perm[None, :]).reshape(-1)
    out = t.clone()
    out[:nqk] = t[idx]
    return out


def apply_rope(x: torch.Tensor, positions: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, rot: int,
               style: str) -> torch.Tensor:
    """x [T, H, D] -> rotated copy (first ``rot`` dims), fp32 math, x.dtype out."""
    xf = x.float()
    c = cos[positions][:, None, :]  # [T,1,rot/2]
    s = sin[positions][:, None, :]
    out = xf.clone()
    if style == "gptj":
        x0 = xf[..., 0:rot:2]
        x1 = xf[..., 1:rot:2]
        out[..., 0:rot:2] = x0 * c - x1 * s
        out[..., 1:rot:2] = x1 * c + x0 * s
    else:
        h = rot // 2
        x0 = xf[..., :h]
        x1 = xf[..., h:rot]
        out[..., :h] = x0 * c - x1 * s
        out[..., h:rot] = x1 * c + x0 * s
    return out.to(x.dtype)


# fp8 KV cache rows: one (token, kv head) row = D e4m3 bytes + a 16-byte tail holding the row's fp32
# scale (bytes D..D+3; D+4..D+15 zero): scale = absmax / 448, value = e4m3 * scale. 16-B aligned rows,
# 0.56x the bytes of a bf16 row at D = 128.
KV8_TAIL = 16


def kv_rows_quant(x: torch.Tensor) -> torch.Tensor:
    """[..., D] float -> [..., D + 16] uint8 fp8 cache rows (csrc kernels: same arithmetic)."""
    xf = x.float()
    D = xf.shape[-1]
    amax = xf.abs().amax(-1, keepdim=True)
    sc = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    q = (xf * (1.0 / sc)).clamp(-448.0, 448.0).to(torch.float8_e4m3fn).view(torch.uint8)
    rows = torch.zeros(*xf.shape[:-1], D + KV8_TAIL, dtype=torch.uint8, device=x.device)
    rows[..., :D] = q
    rows[..., D:D + 4] = sc.contiguous().view(torch.uint8)
    return rows


def kv_rows_dequant(rows: torch.Tensor, D: int) -> torch.Tensor:
    """[..., D + 16] uint8 fp8 cache rows -> [..., D] fp32."""
    q = rows[..., :D].contiguous().view(torch.float8_e4m3fn).float()
    sc = rows[..., D:D + 4].contiguous().view(torch.float32)
    return q * sc


def rope_cache(qkv: torch.Tensor, positions, cos, sin, k_cache, v_cache, slots, nh: int, nkv: int, D: int,
               rot: int, style: str, do_rope: bool = True) -> None:
    """In place: rotate q and k inside qkv; write rotated k and v to the paged cache at slots."""
    T = qkv.shape[0]
    q = qkv[:, : nh * D].view(T, nh, D)
    k = qkv[:, nh * D: (nh + nkv) * D].view(T, nkv, D)
    v = qkv[:, (nh + nkv) * D: (nh + 2 * nkv) * D].view(T, nkv, D)
    if do_rope and rot > 0:
        q.copy_(apply_rope(q, positions, cos, sin, rot, style))
        k.copy_(apply_rope(k, positions, cos, sin, rot, style))
    if k_cache is not None and slots is not None:
        bs = k_cache.shape[2]
        valid = slots >= 0
        sl = slots[valid]
        blk, off = sl // bs, sl % bs
        # cache [num_blocks, nkv, bs, D] (or fp8 rows [.., D + 16] uint8)
        if k_cache.dtype == torch.uint8:
            k_cache[blk, :, off, :] = kv_rows_quant(k[valid])
            v_cache[blk, :, off, :] = kv_rows_quant(v[valid])
        else:
            k_cache[blk, :, off, :] = k[valid].to(k_cache.dtype)
            v_cache[blk, :, off, :] = v[valid].to(v_cache.dtype)


def attn_prefill(qkv: torch.Tensor, cu_seqlens, nh: int, nkv: int, D: int, scale: float) -> torch.Tensor:
    """Causal attention per packed sequence; q/k/v read from the fused qkv rows."""
    T = qkv.shape[0]
    out = torch.empty(T, nh * D, dtype=qkv.dtype, device=qkv.device)
    cu = [int(c) for c in (cu_seqlens.tolist() if torch.is_tensor(cu_seqlens) else cu_seqlens)]
    g = nh // nkv
    for i in range(len(cu) - 1):
        a, b = cu[i], cu[i + 1]
        if b == a:
            continue
        q = qkv[a:b, : nh * D].view(b - a, nh, D).float().transpose(0, 1)
        k = qkv[a:b, nh * D: (nh + nkv) * D].view(b - a, nkv, D).float().transpose(0, 1)
        v = qkv[a:b, (nh + nkv) * D: (nh + 2 * nkv) * D].view(b - a, nkv, D).float().transpose(0, 1)
        k = k.repeat_interleave(g, 0)
        v = v.repeat_interleave(g, 0)
        s = torch.matmul(q, k.transpose(1, 2)) * scale
        mask = torch.ones(b - a, b - a, dtype=torch.bool, device=qkv.device).tril()
        s = s.masked_fill(~mask, float("-inf"))
        p = torch.softmax(s, -1)
        o = torch.matmul(p, v).transpose(0, 1).reshape(b - a, nh * D)
        out[a:b] = o.to(qkv.dtype)
    return out


def gather_kv(cache: torch.Tensor, block_table_row: torch.Tensor, ctx: int) -> torch.Tensor:
    """Paged cache [nb, nkv, bs, D] -> contiguous [nkv, ctx, D] for one sequence (fp8 rows dequantised
    to fp32)."""
    bs = cache.shape[2]
    nblk = (ctx + bs - 1) // bs
    blocks = cache[block_table_row[:nblk].long()]  # [nblk, nkv, bs, D]
    out = blocks.permute(1, 0, 2, 3).reshape(cache.shape[1], nblk * bs, cache.shape[3])[:, :ctx]
    return kv_rows_dequant(out, cache.shape[3] - KV8_TAIL) if cache.dtype == torch.uint8 else out


def attn_decode(q: torch.Tensor, k_cache, v_cache, block_tables, ctx_lens, nh: int, nkv: int, D: int,
                scale: float) -> torch.Tensor:
    """q [B, >= nh*D] (row-strided view allowed); returns [B, nh*D]."""
    B = q.shape[0]
    g = nh // nkv
    out = torch.empty(B, nh * D, dtype=q.dtype, device=q.device)
    for b in range(B):
        ctx = int(ctx_lens[b])
        qq = q[b, : nh * D].view(nh, D).float()
        if ctx == 0:
            out[b] = 0
            continue
        k = gather_kv(k_cache, block_tables[b], ctx).float().repeat_interleave(g, 0)  # [nh, ctx, D]
        v = gather_kv(v_cache, block_tables[b], ctx).float().repeat_interleave(g, 0)
        s = torch.einsum("hd,htd->ht", qq, k) * scale
        p = torch.softmax(s, -1)
        out[b] = torch.einsum("ht,htd->hd", p, v).reshape(-1).to(q.dtype)
    return out


def attn_extend(q: torch.Tensor, k_cache, v_cache, block_tables, cu_q, ctx_lens, nh: int, nkv: int, D: int,
                scale: float, window: int = 0) -> torch.Tensor:
    """Chunked prefill over the paged cache: sequence b's rows cu_q[b]:cu_q[b+1] sit at positions
    ctx_lens[b] - qlen ... ctx_lens[b] - 1 and attend every cached key up to their own position."""
    T = q.shape[0]
    g = nh // nkv
    out = torch.zeros(T, nh * D, dtype=q.dtype, device=q.device)
    cu = [int(c) for c in cu_q.tolist()]
    for b in range(len(cu) - 1):
        a, e = cu[b], cu[b + 1]
        if e == a:
            continue
        ctx = int(ctx_lens[b])
        p0 = ctx - (e - a)
        qq = q[a:e, : nh * D].view(e - a, nh, D).float().transpose(0, 1)  # [nh, q, D]
        k = gather_kv(k_cache, block_tables[b], ctx).float().repeat_interleave(g, 0)  # [nh, ctx, D]
        v = gather_kv(v_cache, block_tables[b], ctx).float().repeat_interleave(g, 0)
        s = torch.matmul(qq, k.transpose(1, 2)) * scale
        qpos = torch.arange(p0, ctx, device=q.device)[:, None]
        kpos = torch.arange(ctx, device=q.device)[None, :]
        s = s.masked_fill((kpos > qpos) | ((kpos <= qpos - window) if window > 0 else False), float("-inf"))
        out[a:e] = torch.matmul(torch.softmax(s, -1), v).transpose(0, 1).reshape(e - a, nh * D).to(q.dtype)
    return out


def glu_split(w_or_y: torch.Tensor, dim: int = -1):
    """Split a 16-row/column interleaved gate|up tensor into (gate, up)."""
    n = w_or_y.shape[dim]
    shp = list(w_or_y.shape)
    d = dim % len(shp)
    v = w_or_y.reshape(shp[:d] + [n // 32, 2, 16] + shp[d + 1:])
    gate = v.select(d + 1, 0).reshape(shp[:d] + [n // 2] + shp[d + 1:])
    up = v.select(d + 1, 1).reshape(shp[:d] + [n // 2] + shp[d + 1:])
    return gate, up


def glu_interleave(gate: torch.Tensor, up: torch.Tensor, dim: int = 0) -> torch.Tensor:
    """Inverse of :func:`glu_split`: [F, ...] x2 -> [2F, ...] interleaved in 16-row groups."""
    d = dim % gate.dim()
    F_ = gate.shape[d]
    if F_ % 16:
        raise ValueError("gated MLP width must be a multiple of 16 per rank")
    shp = list(gate.shape)
    g = gate.reshape(shp[:d] + [F_ // 16, 1, 16] + shp[d + 1:])
    u = up.reshape(shp[:d] + [F_ // 16, 1, 16] + shp[d + 1:])
    return torch.cat([g, u], dim=d + 1).reshape(shp[:d] + [2 * F_] + shp[d + 1:])


def dequant_fp8(w_q: torch.Tensor, w_scale: torch.Tensor, dtype=torch.float32) -> torch.Tensor:
    return (w_q.view(torch.float8_e4m3fn).float() * w_scale.float()[:, None]).to(dtype)


def fake_quant_fp8_act(x: torch.Tensor) -> torch.Tensor:
    """Per-token e4m3 fake quantisation of GEMM activations, as the W8A8 path quantises them (csrc/quant.hip
    quant_fp8_rows_ld, the add_norm / attention fp8 twins): scale = absmax(row) / 448 (1 for a zero row),
    q = e4m3(clamp(x * (1 / scale), +-448)); returns q * scale in fp32."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1, keepdim=True)
    s = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    q = (xf * (1.0 / s)).clamp(-448, 448).to(torch.float8_e4m3fn).float()
    return q * s


def quant_mx_fp8(x: torch.Tensor):
    """OCP MX-fp8 of rows, as a W8A8 SwiGLU epilogue writes it for the down projection (csrc/common.h
    img_store_rows, mx_block_exp): per row and 32 columns the e8m0 scale 2^e with the smallest e such that the block's
    |max| / 2^e <= 448 (e clamped to [-126, 126]; 0 for an all-zero block), q = e4m3(x / 2^e). Returns (q uint8
    [M, K], s uint8 [M, K / 32] = e + 127)."""
    M, K = x.shape
    xb = x.float().reshape(M, K // 32, 32)
    amax = xb.abs().amax(-1)
    bits = (amax / 448.0).view(torch.int32)
    e = ((bits >> 23) & 255) - 127 + ((bits & 0x7FFFFF) != 0).to(torch.int32)
    e = torch.where(amax > 0, e.clamp(-126, 126), torch.zeros_like(e))
    q = (xb * torch.ldexp(torch.ones_like(amax), -e)[..., None]).clamp(-448, 448).to(torch.float8_e4m3fn)
    return q.view(torch.uint8).reshape(M, K), (e + 127).to(torch.uint8)


def dequant_mx_fp8(q: torch.Tensor, s: torch.Tensor) -> torch.Tensor:
    M, K = q.shape
    qf = q.view(torch.float8_e4m3fn).float().reshape(M, K // 32, 32)
    return (qf * torch.ldexp(torch.ones(s.shape), s.to(torch.int32) - 127)[..., None]).reshape(M, K)


def fake_quant_mx_act(x: torch.Tensor) -> torch.Tensor:
    """MX-fp8 fake quantisation (quant_mx_fp8 then back to fp32)."""
    return dequant_mx_fp8(*quant_mx_fp8(x))


def linear(x: torch.Tensor, w: torch.Tensor, bias=None, act: str = "none", glu: bool = False,
           w_scale: Optional[torch.Tensor] = None, a8=False) -> torch.Tensor:
    """``a8`` (fp8 weights only): per-token e4m3 activations as well - the fp32 fake-quant oracle of W8A8;
    ``a8="mx"``: MX-fp8 activations (per-32 e8m0 block scales)."""
    wf = dequant_fp8(w, w_scale) if w_scale is not None else w.float()
    if a8 and w_scale is not None:
        xf = fake_quant_mx_act(x) if a8 == "mx" else fake_quant_fp8_act(x)
    else:
        xf = x.float()
    y = xf @ wf.t()
    if bias is not None:
        y = y + bias.float()
    if glu:
        g, u = glu_split(y, -1)
        y = F.silu(g) * u
    else:
        y = _act(y, act)
    return y.to(x.dtype)


def quant_fp8_rows(w: torch.Tensor):
    wf = w.float()
    amax = wf.abs().amax(dim=1).clamp_min(0)
    scale = torch.where(amax > 0, amax / 448.0, torch.ones_like(amax))
    q = (wf / scale[:, None]).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8)
    return q, scale


# ---------------------------------------------------------------------------------------- sampling
# CPU definition of the GPU sampler (csrc/sampling.hip sample_v3 / sample_cand): temperature ->
# top-k -> top-p -> Gumbel-max with Philox-4x32-10 noise keyed by (row seed, global token index).
# Top-p mass is summed as 2^-32 fixed-point integers, so the kept set does not depend on summation
# order - which is what lets a vocab-parallel (candidate) evaluation reproduce the full-row result.
def philox(idx: np.ndarray, seed: int) -> np.ndarray:
    """Philox-4x32-10 first output word for counters (idx, 0, 0, 0) and key = 64-bit seed."""
    m = np.uint64(0xFFFFFFFF)
    c0 = idx.astype(np.uint64) & m
    c1 = np.zeros_like(c0)
    c2 = np.zeros_like(c0)
    c3 = np.zeros_like(c0)
    k0, k1 = np.uint64(seed & 0xFFFFFFFF), np.uint64((seed >> 32) & 0xFFFFFFFF)
    for _ in range(10):
        p0 = np.uint64(0xD2511F53) * c0
        p1 = np.uint64(0xCD9E8D57) * c2
        h0, l0, h1, l1 = p0 >> np.uint64(32), p0 & m, p1 >> np.uint64(32), p1 & m
        c0, c1, c2, c3 = (h1 ^ c1 ^ k0) & m, l1, (h0 ^ c3 ^ k1) & m, l0
        k0, k1 = (k0 + np.uint64(0x9E3779B9)) & m, (k1 + np.uint64(0xBB67AE85)) & m
    return c0


def _mass(x: np.ndarray, mx: np.float32) -> np.ndarray:
    return (np.exp((x - mx).astype(np.float32)).astype(np.float32) * np.float32(4294967296.0)).astype(np.uint64)


def _select(x: np.ndarray, idx: np.ndarray, t: float, k: int, p: float, seed: int, V: int) -> int:
    """One row: x = scaled logits of the (candidate) elements, idx their global token ids."""
    valid = np.isfinite(x) | (x > -np.inf)
    x, idx = x[valid], idx[valid]
    if x.size == 0:
        return 0
    greedy = not t > 0 or k == 1
    thr = -np.inf
    if not greedy:
        order = np.lexsort((idx, -x))  # value desc, index asc
        xs = x[order]
        mx = np.float32(xs[0])
        if 0 < k < V and k <= xs.size:
            thr = xs[k - 1]
        if p < 1.0:
            kept = xs[xs >= thr]
            m = _mass(kept, mx)
            z = int(m.sum(dtype=np.uint64))
            target = max(1, int(float(p) * float(z)))
            cum = np.cumsum(m, dtype=np.uint64)
            j = int(np.searchsorted(cum, np.uint64(target), side="left"))
            tp = kept[min(j, kept.size - 1)]
            thr = max(thr, tp)
    v = x.astype(np.float32)
    if not greedy:
        keep = x >= thr
        v, idx = v[keep], idx[keep]
        r = philox(idx, seed)
        u = ((r >> np.uint64(8)).astype(np.float32) + np.float32(0.5)) * np.float32(1.0 / 16777216.0)
        v = (v - np.log(-np.log(u))).astype(np.float32)
    best = v.max()
    return int(idx[v == best].min())


def sample(logits: torch.Tensor, temperature, top_k, top_p, seeds, generator=None) -> torch.Tensor:
    """Full-row sampler (the GPU ``sample_v3`` definition): temperature -> top-k -> top-p -> Gumbel-max."""
    B, V = logits.shape
    lg = logits.detach().float().cpu().numpy()
    out = torch.empty(B, dtype=torch.long)
    for b in range(B):
        t = float(temperature[b]) if temperature is not None else 0.0
        k = int(top_k[b]) if top_k is not None else 0
        p = float(top_p[b]) if top_p is not None else 1.0
        sc = np.float32(1.0) if (not t > 0 or k == 1) else np.float32(1.0) / np.float32(t)
        x = lg[b].astype(np.float32) * sc
        seed = int(seeds[b]) & ((1 << 64) - 1) if seeds is not None else 0
        out[b] = _select(x, np.arange(V), t, k, p, seed, V)
    return out.to(logits.device)


def cand_topk(local: torch.Tensor, lo: int, V: int, temperature, top_k, K: int, KC: int) -> torch.Tensor:
    """Per-rank candidates of a vocab shard (GPU ``cand_topk``): every element whose scaled logit is
    >= the shard's K-th largest, packed per row as [KC values | KC global indices as int32 bits]."""
    B, vl = local.shape
    lg = local.detach().float().cpu().numpy()
    pack = np.zeros((B, 2 * KC), dtype=np.float32)
    for b in range(B):
        t = float(temperature[b]) if temperature is not None else 0.0
        k = int(top_k[b]) if top_k is not None else 0
        sc = np.float32(1.0) if (not t > 0 or k == 1) else np.float32(1.0) / np.float32(t)
        n = max(0, min(vl, V - lo))
        x = lg[b, :n].astype(np.float32) * sc
        kth = np.sort(x)[::-1][K - 1] if n >= K else -np.inf
        sel = np.flatnonzero(x >= kth)[:KC]
        vals = np.full(KC, -np.inf, dtype=np.float32)
        ids = np.full(KC, 0x7FFFFFFF, dtype=np.int32)
        vals[:sel.size] = x[sel]
        ids[:sel.size] = lo + sel
        pack[b, :KC] = vals
        pack[b, KC:] = ids.view(np.float32)
    return torch.from_numpy(pack).to(local.device)


def sample_cand(pack: torch.Tensor, groups: int, KC: int, temperature, top_k, top_p, seeds, V: int) -> torch.Tensor:
    """Sampling over gathered candidates [B, groups * 2KC] (GPU ``sample_cand``)."""
    B = pack.shape[0]
    a = pack.detach().cpu().numpy().reshape(B, groups, 2, KC)
    out = torch.empty(B, dtype=torch.long)
    for b in range(B):
        x = a[b, :, 0, :].reshape(-1).astype(np.float32)
        idx = a[b, :, 1, :].reshape(-1).view(np.int32).astype(np.int64)
        t = float(temperature[b]) if temperature is not None else 0.0
        k = int(top_k[b]) if top_k is not None else 0
        p = float(top_p[b]) if top_p is not None else 1.0
        seed = int(seeds[b]) & ((1 << 64) - 1) if seeds is not None else 0
        out[b] = _select(x, idx, t, k, p, seed, V)
    return out.to(pack.device)


def cross_entropy(logits: torch.Tensor, labels: torch.Tensor) -> torch.Tensor:
    """Shifted LM loss as in the reference (gptj_modeling.py:612-622)."""
    return F.cross_entropy(logits[..., :-1, :].reshape(-1, logits.shape[-1]).float(),
                           labels[..., 1:].reshape(-1), ignore_index=-100)


def softmax_scale(D: int) -> float:
    return 1.0 / math.sqrt(D)


# ------------------------------------------------------------------- fp32 residual stream / latent attention / MoE
# CPU definitions of the kernels in csrc/resid32.hip, gemm_any.hip, attention_latent.hip and moe.hip: fp32 math,
# results rounded to the storage type at the same places as on the GPU.
def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    """fp32 rows table[ids] * scale."""
    return table[ids.clamp(0, table.shape[0] - 1)].float() * scale


def resid_add_norm(x: torch.Tensor, a, b, w, woff: float, eps: float, out_dtype, want_y: bool = True):
    """x (fp32, in place) += (a + b) for the addends given; returns rms_norm(x) * (woff + w) in ``out_dtype``
    (None when ``want_y`` is false)."""
    if a is not None or b is not None:
        d = a.float() if a is not None else None
        if b is not None:
            d = b.float() if d is None else d + b.float()
        x.add_(d)
    if not want_y:
        return None
    y = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * (woff + w.float())
    return y.to(out_dtype)


def linear_f(x: torch.Tensor, w: torch.Tensor, out_dtype) -> torch.Tensor:
    """x [M, K] . w [N, K]^T with fp32 accumulation -> [M, N] in ``out_dtype``."""
    return (x.float() @ w.float().t()).to(out_dtype)


def head_absorb(q: torch.Tensor, uk_t: torch.Tensor, out_dtype=torch.float32, extra: int = 0) -> torch.Tensor:
    """qa[t, h, r] = sum_d q[t, h * (dim + extra) + d] * uk_t[h, r, d] -> [T, H, R + extra] (uk_t: the key
    up-projection, per head transposed to [R, dim]). ``extra`` > 0: every head of q carries that many more numbers
    after its ``dim``, and the result that many more columns after R, left for the caller to fill."""
    H, R, dim = uk_t.shape
    T = q.shape[0]
    qh = q[:, : H * (dim + extra)].float().reshape(T, H, dim + extra)[..., :dim]
    qa = torch.zeros(T, H, R + extra, dtype=out_dtype, device=q.device)
    qa[..., :R] = torch.einsum("thd,hrd->thr", qh, uk_t.float()).to(out_dtype)
    return qa


def latent_qa_dtype(cache) -> torch.dtype:
    return torch.float32


def head_expand(o: torch.Tensor, uv: torch.Tensor, out_dtype) -> torch.Tensor:
    """y[t, h * vd + v] = sum_r o[t, h, r] * uv[h * vd + v, r] -> [T, H * vd] in ``out_dtype``; columns of ``o``
    beyond uv's width are not read."""
    T, H, _ = o.shape
    R = uv.shape[1]
    return torch.einsum("thr,hvr->thv", o[..., :R].float(), uv.float().view(H, -1, R)).reshape(T, -1).to(out_dtype)


def _turn_neighbours(x: torch.Tensor, cs: torch.Tensor) -> torch.Tensor:
    """x [T, ..., rot] with the pairs (2i, 2i + 1), i < cs.shape[1], turned by cs [T, dims / 2, 2] = (cos, sin); the
    numbers from ``dims`` on pass unchanged."""
    T, dims = x.shape[0], 2 * cs.shape[1]
    shape = [T] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = cs[..., 0].view(shape), cs[..., 1].view(shape)
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    turned = torch.stack([u * c - v * s, v * c + u * s], -1).reshape(*x.shape[:-1], dims)
    return torch.cat([turned, x[..., dims:]], -1)


def latent_norm_cache(src: torch.Tensor, off: int, R: int, w: torch.Tensor, eps: float, cache: torch.Tensor,
                      slots: torch.Tensor, rot: int = 0, cs: Optional[torch.Tensor] = None,
                      qa: Optional[torch.Tensor] = None, off_q: int = 0, qdim: int = 0) -> None:
    """cache[slot[t], :R] = rms_norm(src[t, off : off + R]) * w (slots < 0 are skipped); cache is [blocks, bs,
    R + rot]. ``rot`` > 0: the ``rot`` columns after the latent's are one key part shared by all heads; turned by
    ``cs`` [T, dims / 2, 2] (neighbouring pairs of the first ``dims`` <= rot numbers) they fill the cached row, and every query head's last ``rot`` numbers
    (head h at src[t, off_q + h * (qdim + rot) + qdim]), turned the same way, fill qa[t, h, R:]."""
    c = src[:, off:off + R].float()
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    if rot:
        c = torch.cat([c, _turn_neighbours(src[:, off + R:off + R + rot].float(), cs)], -1)
        T, H = qa.shape[0], qa.shape[1]
        qr = src[:, off_q:off_q + H * (qdim + rot)].float().reshape(T, H, qdim + rot)[..., qdim:]
        qa[..., R:] = _turn_neighbours(qr, cs).to(qa.dtype)
    valid = slots >= 0
    cache.view(-1, R + rot)[slots[valid]] = c[valid].to(cache.dtype)


def rope_angles(positions: torch.Tensor, freqs: torch.Tensor) -> torch.Tensor:
    """fp32 [T, len(freqs), 2] = (cos, sin) of position * freqs[i], the product rounded to fp32."""
    ang = positions.to(torch.float32)[:, None] * freqs.float()[None, :]
    return torch.stack([torch.cos(ang), torch.sin(ang)], -1)


def latent_attn(qa: torch.Tensor, cache: torch.Tensor, block_tables, cu_q, ctx_lens, window: int,
                scale: float, max_qlen: int = 0, max_ctx: int = 0) -> torch.Tensor:
    """Multi-query attention whose keys and values are the cached latent rows (csrc/attention_latent.hip):
    qa fp32 [T, H, R]; sequence b's rows cu_q[b]:cu_q[b+1] sit at positions ctx_lens[b] - qlen .. ctx_lens[b] - 1
    and see the positions j with 0 <= i - j (< window when window > 0). Returns fp32 [T, H, R]."""
    T, H, R = qa.shape
    bs = cache.shape[1]
    out = torch.zeros(T, H, R, dtype=torch.float32, device=qa.device)
    cu = [int(c) for c in cu_q.tolist()]
    for b in range(len(cu) - 1):
        a, e = cu[b], cu[b + 1]
        ctx = int(ctx_lens[b])
        if e == a or ctx <= 0:
            continue
        p0 = ctx - (e - a)
        nblk = -(-ctx // bs)
        c = cache[block_tables[b, :nblk].long()].reshape(nblk * bs, R)[:ctx].float()
        s = torch.einsum("thr,jr->htj", qa[a:e].float() * scale, c)
        i = torch.arange(p0, ctx, device=qa.device)[:, None]
        j = torch.arange(ctx, device=qa.device)[None, :]
        vis = (i - j >= 0)
        if window > 0:
            vis &= (i - j < window)
        s = s.masked_fill(~vis, float("-inf"))
        out[a:e] = torch.einsum("htj,jr->thr", torch.softmax(s, -1), c)
    return out


def glu_clamped(g: torch.Tensor, u: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return g * torch.sigmoid(alpha * g) * (u + 1)


def glu_clamp(gu: torch.Tensor, F_: int, limit: float, alpha: float) -> torch.Tensor:
    """[T, 2F] gate | up halves -> [T, F]."""
    return glu_clamped(gu[:, :F_].float(), gu[:, F_:2 * F_].float(), limit, alpha).to(gu.dtype)


def moe_route(z: torch.Tensor, corr: Optional[torch.Tensor], top: int, normalize: bool = True):
    """fp32 router logits [T, E] -> (idx int32 [T, top], weights fp32 [T, top]): scores sigmoid(z), the ``top``
    largest of score + corr chosen (ties: lower index), weights = chosen scores / (their sum + 1e-20), or the chosen
    scores themselves (``normalize`` false)."""
    s = torch.sigmoid(z.float())
    ch = s if corr is None else s + corr.float()
    # descending by value, ascending by index among equals
    order = torch.argsort(ch, dim=-1, descending=True, stable=True)
    idx = order[:, :top]
    w = torch.gather(s, 1, idx)
    if normalize:
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
    return idx.to(torch.int32), w


def moe_router(h: torch.Tensor, router: torch.Tensor, corr: Optional[torch.Tensor], top: int,
               normalize: bool = True):
    """Router logits in fp32 from the layer input, then :func:`moe_route`."""
    return moe_route(linear_f(h, router, torch.float32), corr, top, normalize)


def moe_experts(h: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, gate: torch.Tensor, up: torch.Tensor,
                down: torch.Tensor, limit: float, alpha: float, shared: Optional[torch.Tensor] = None,
                combine: bool = True, act: str = "glu_clamp", weight_input: bool = False) -> torch.Tensor:
    """sum_j wts[t, j] * down_e(glu(gate_e h, up_e h)) (+ shared) with e = idx[t, j] -> fp32 [T, N]. Stacked expert
    weights gate / up [E, F, K], down [E, N, F]; the activation is rounded to the storage type between the
    products, as the grouped GEMMs do. ``act`` "silu": silu(g) * u without clamps. ``weight_input``: the weight
    multiplies the expert's input instead, sum_j down_e(act(w gate_e h, w up_e h)) (experts have no biases, so the
    weight is applied to the two products)."""
    T = h.shape[0]
    N = down.shape[1]
    out = torch.zeros(T, N, dtype=torch.float32, device=h.device)
    hf = h.float()
    for j in range(idx.shape[1]):
        for e in idx[:, j].unique().tolist():
            rows = torch.nonzero(idx[:, j] == e).flatten()
            x = hf[rows]
            g_, u_ = x @ gate[e].float().t(), x @ up[e].float().t()
            if weight_input:
                g_, u_ = g_ * wts[rows, j:j + 1], u_ * wts[rows, j:j + 1]
            a = (g_ * torch.sigmoid(g_) * u_ if act == "silu" else glu_clamped(g_, u_, limit, alpha)).to(h.dtype).float()
            out[rows] += (a @ down[e].float().t()) * (1.0 if weight_input else wts[rows, j:j + 1])
    if shared is not None:
        out += shared.float()
    return out


# ----------------------------------- residual streams / convolution tails / matrix-state recurrences / sink attention
def _seq_rows(cu, ctx_lens):
    """(b, first row, rows, first position) of every sequence of a step with rows."""
    cu_l, cl = cu.tolist(), ctx_lens.tolist()
    return [(b, cu_l[b], cu_l[b + 1] - cu_l[b], cl[b] - (cu_l[b + 1] - cu_l[b])) for b in range(len(cu_l) - 1)
            if cu_l[b + 1] > cu_l[b] and cl[b] > 0]


def embed_streams(ids, positions, table, pos_table, streams: int) -> torch.Tensor:
    """fp32 [streams, T, W]: every stream starts as table[ids] (+ pos_table[positions])."""
    x = table[ids.clamp(0, table.shape[0] - 1)].float()
    if pos_table is not None:
        x = x + pos_table[positions.clamp(0, pos_table.shape[0] - 1)].float()
    return x.unsqueeze(0).repeat(streams, 1, 1).contiguous()


def stream_add_norm(x, y, mix, outw, c: float, inw, w, eps: float, rms: bool, out_dtype):
    """x fp32 [S, T, W], updated in place when ``y`` is given: x_s <- sum_r mix[r, s] x_r + c * outw[s] * y.
    With ``w``: returns norm(sum_s inw[s] x_s) * w in ``out_dtype`` (inw None: the plain sum; rms False: mean
    subtracted, variance = mean squared deviation)."""
    if y is not None:
        x.copy_(torch.einsum("rs,rtw->stw", mix, x) + (c * outw)[:, None, None] * y.float()[None])
    if w is None:
        return None
    u = x.sum(0) if inw is None else torch.einsum("s,stw->tw", inw, x)
    if not rms:
        u = u - u.mean(-1, keepdim=True)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def causal_conv(x, w, state, cu, ctx_lens, state_slots, residual: bool, silu: bool, out_dtype, bias=None):
    """Per-channel causal convolution over time of x [T, C] with w [C, taps] (last column: the current row), each
    sequence continuing from the taps - 1 inputs in its state slot (state fp32 [slots, taps - 1, C], renewed here;
    a portion starting at position 0 reads zeros). ``residual`` adds x itself; ``bias`` [C] is added to every row;
    ``silu`` applies x * sigmoid(x)."""
    T, C = x.shape
    taps = w.shape[1]
    R = taps - 1
    out = torch.zeros(T, C, dtype=torch.float32)
    wf = w.float()
    slots = state_slots.tolist()
    for b, t0, q, p0 in _seq_rows(cu, ctx_lens):
        cur = x[t0:t0 + q].float()
        if R:
            tail = state[slots[b]].clone() if p0 > 0 else torch.zeros(R, C)
            if p0 < R:
                tail[:R - p0] = 0
            full = torch.cat([tail, cur], 0)
            state[slots[b]] = full[-R:]
        else:
            full = cur
        y = sum(wf[:, k] * full[k:k + q] for k in range(taps))
        if residual:
            y = y + cur
        if bias is not None:
            y = y + bias.float()
        out[t0:t0 + q] = y
    if silu:
        out = out * torch.sigmoid(out)
    return out.to(out_dtype)


def gated_group_norm(o, gate, w, eps: float, act: str, c: float, out=None, out_dtype=None, groups: int = 0,
                     gate_first: bool = False):
    """o fp32 [T, groups * n] divided per group of n = len(w) by its root mean square, times w, times act(gate)
    (``sigmoid`` or ``silu``), times c; written to ``out`` (a [T, groups * n] view) when given. ``groups`` > 0: w
    holds a weight for every column ([groups * n]) instead of one per column of a group. ``gate_first``: the gate is
    applied before the norm, rms_div(o * act(gate)) * w."""
    T, N = o.shape
    n = N // groups if groups else w.numel()
    g = gate.float()
    a = torch.sigmoid(g) if act == "sigmoid" else g * torch.sigmoid(g)
    of = o.float() * a if gate_first else o.float()
    og = of.view(T, N // n, n)
    y = og * torch.rsqrt(og.pow(2).mean(-1, keepdim=True) + eps)
    y = (y.view(T, N) * w.float() if groups else (y * w.float()).view(T, N)) * c
    if not gate_first:
        y = y * a
    if out is not None:
        out.copy_(y)
        return out
    return y.to(out_dtype)


def act_fn(x, act: str, params=()):
    """Ungated activation of every number of x, in fp32, result in x's type. ``gelu_tanh``, ``silu``, or ``xielu``
    with params (a, b): z > 0: a z^2 + z / 2; z <= 0: b (exp(z) - 1 - z) + z / 2."""
    z = x.float()
    if act == "xielu":
        a, b = params
        y = torch.where(z > 0, a * z * z + 0.5 * z, b * (torch.expm1(z) - z) + 0.5 * z)
    elif act == "gelu_tanh":
        y = torch.nn.functional.gelu(z, approximate="tanh")
    else:
        y = z * torch.sigmoid(z)
    return y.to(x.dtype)


def glu_act(gu, F_: int, act: str):
    """act(gu[:, :F]) * gu[:, F:2F]; act ``gelu_tanh`` or ``silu``."""
    g, u = gu[:, :F_].float(), gu[:, F_:2 * F_].float()
    a = torch.nn.functional.gelu(g, approximate="tanh") if act == "gelu_tanh" else g * torch.sigmoid(g)
    return (a * u).to(gu.dtype)


def decay_recurrence(q, k, v, decay, state, cu, ctx_lens, state_slots, heads: int, dim: int, vdim: int,
                     silu_in: bool = True):
    """Per head S <- decay_h S + k v^T, o = S^T q over each sequence's rows, S fp32 [slots, heads, dim, vdim]
    carried in the sequence's slot (zero when the portion starts at position 0). Returns fp32 [T, heads * vdim]."""
    T = q.shape[0]
    out = torch.zeros(T, heads * vdim, dtype=torch.float32)
    slots = state_slots.tolist()

    def pre(t):
        t = t.float()
        return t * torch.sigmoid(t) if silu_in else t
    for b, t0, n, p0 in _seq_rows(cu, ctx_lens):
        S = state[slots[b]].clone() if p0 > 0 else torch.zeros(heads, dim, vdim)
        qq = pre(q[t0:t0 + n]).view(n, heads, dim)
        kk = pre(k[t0:t0 + n]).view(n, heads, dim)
        vv = pre(v[t0:t0 + n]).view(n, heads, vdim)
        for j in range(n):
            S = decay[:, None, None] * S + kk[j, :, :, None] * vv[j, :, None, :]
            out[t0 + j] = torch.einsum("hdv,hd->hv", S, qq[j]).reshape(-1)
        state[slots[b]] = S
    return out


def delta_recurrence(q, k, v, a, b_, A_log, dt_bias, state, cu, ctx_lens, state_slots, heads: int, kv_heads: int,
                     dim: int, vdim: int):
    """Gated delta rule per head: S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, with k and q made unit
    vectors (1e-6 inside the root), q also divided by sqrt(dim), beta = sigmoid(b), g = exp(-exp(A_log)
    softplus(a + dt_bias)). q, k [T, kv_heads * dim], v [T, heads * vdim], a, b_ [T, heads]. fp32 out."""
    T = q.shape[0]
    rep = heads // kv_heads
    out = torch.zeros(T, heads * vdim, dtype=torch.float32)
    slots = state_slots.tolist()
    for b, t0, n, p0 in _seq_rows(cu, ctx_lens):
        S = state[slots[b]].clone() if p0 > 0 else torch.zeros(heads, dim, vdim)
        qq = q[t0:t0 + n].float().view(n, kv_heads, dim)
        kk = k[t0:t0 + n].float().view(n, kv_heads, dim)
        qq = (qq * torch.rsqrt(qq.pow(2).sum(-1, keepdim=True) + 1e-6) * dim ** -0.5).repeat_interleave(rep, 1)
        kk = (kk * torch.rsqrt(kk.pow(2).sum(-1, keepdim=True) + 1e-6)).repeat_interleave(rep, 1)
        vv = v[t0:t0 + n].float().view(n, heads, vdim)
        beta = torch.sigmoid(b_[t0:t0 + n].float())
        g = torch.exp(-torch.exp(A_log.float()) * torch.nn.functional.softplus(a[t0:t0 + n].float() + dt_bias.float()))
        for j in range(n):
            S = g[j][:, None, None] * S
            u = beta[j][:, None] * (vv[j] - torch.einsum("hdv,hd->hv", S, kk[j]))
            S = S + kk[j][:, :, None] * u[:, None, :]
            out[t0 + j] = torch.einsum("hdv,hd->hv", S, qq[j]).reshape(-1)
        state[slots[b]] = S
    return out


def rope_angle_table(npos: int, dims: int, base: float, scaling=None) -> torch.Tensor:
    """fp32 [npos, dims / 2, 2] = (cos, sin) of position * f_i, f_i = base^(-2 i / dims). ``scaling`` = (factor,
    original, fast, slow): frequencies between the two turn counts are blended towards f_i / factor (YaRN) and both
    cos and sin are multiplied by 0.1 ln(factor) + 1. Angles are formed in float64 and rounded once."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float64)
    amp = 1.0
    if scaling is not None:
        factor, original, fast, slow = scaling

        def turn_dim(turns):
            return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
        lo = max(math.floor(turn_dim(fast)), 0)
        hi = min(math.ceil(turn_dim(slow)), dims - 1)
        ramp = ((torch.arange(half, dtype=torch.float64) - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        amp = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(npos, dtype=torch.float64)[:, None] * f[None, :]
    return torch.stack([torch.cos(ang) * amp, torch.sin(ang) * amp], -1).float().contiguous()


def rope_bias_cache(proj, off_q: int, off_k: int, off_v: int, bias, positions, table, rot: int, k_cache, v_cache,
                    slots, heads: int, kv_heads: int, dim: int, vdim: int):
    """From the projection rows: q (+ bias) and k (+ bias) with their first ``rot`` dimensions per head turned by
    ``table`` (i paired with i + rot / 2), v (+ bias). Returns q fp32 [T, heads * dim]; k / v go into the paged
    caches [blocks, block_size, kv_heads * dim | kv_heads * vdim] at ``slots`` (< 0: not cached)."""
    T = proj.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    q, k, v = (proj[:, o:o + n].float() for o, n in ((off_q, nq), (off_k, nk), (off_v, nv)))
    if bias is not None:
        bf = bias.float()
        q, k, v = q + bf[:nq], k + bf[nq:nq + nk], v + bf[nq + nk:]
    half = rot // 2
    if half:
        cs = table[positions.clamp(0, table.shape[0] - 1)]  # [T, half, 2]
        c, s = cs[:, None, :, 0], cs[:, None, :, 1]

        def turn(x, n):
            x = x.view(T, n, dim)
            a, b = x[..., :half], x[..., half:rot]
            return torch.cat([a * c - b * s, b * c + a * s, x[..., rot:]], -1).reshape(T, n * dim)
        q, k = turn(q, heads), turn(k, kv_heads)
    keep = slots >= 0
    k_cache.view(-1, nk)[slots[keep]] = k[keep].to(k_cache.dtype)
    v_cache.view(-1, nv)[slots[keep]] = v[keep].to(v_cache.dtype)
    return q.contiguous()


def sink_attn(q, k_cache, v_cache, block_tables, cu, ctx_lens, heads: int, kv_heads: int, dim: int, vdim: int,
              scale: float, softcap: float, all_groups: bool, max_qlen: int = 0, num_decode: int = 0,
              sink: bool = True, chunk: int = 0, vshare: int = 1, precise: bool = False):
    """Causal attention of every row over its sequence's cached keys with a sink in the softmax denominator
    (p_j = exp(s_j) / (1 + sum exp(s)); ``sink`` false: the ordinary softmax) and optionally soft-capped scores.
    ``chunk`` > 0: a row at position i sees only the keys from floor(i / chunk) * chunk on. ``vshare`` > 1: that many
    neighbouring key heads read the same value head (the value cache holds kv_heads / vshare heads). Returns fp32
    [T, heads, R]: head h's weights applied to the value rows of every group side by side (``all_groups``,
    R = kv_heads / vshare * vdim) or of its own group only (R = vdim). ``max_qlen`` (longest portion) and
    ``num_decode`` (leading single-row sequences) and ``precise`` (32-bit queries and weights on the matrix cores)
    only steer the GPU kernels."""
    T = q.shape[0]
    bs = k_cache.shape[1]
    rep = heads // kv_heads
    vh = kv_heads // vshare
    R = vh * vdim if all_groups else vdim
    out = torch.zeros(T, heads, R, dtype=torch.float32)
    for b, t0, n, p0 in _seq_rows(cu, ctx_lens):
        L = p0 + n
        blocks = block_tables[b, : -(-L // bs)].long()
        K = k_cache[blocks].reshape(-1, kv_heads, dim)[:L].float()
        V = v_cache[blocks].reshape(-1, vh, vdim)[:L].float().repeat_interleave(vshare, 1)
        qq = q[t0:t0 + n].view(n, heads, dim).float()
        s = torch.einsum("nhd,lhd->hnl", qq, K.repeat_interleave(rep, 1)) * scale
        if softcap:
            s = softcap * torch.tanh(s / softcap)
        rows = (p0 + torch.arange(n))[:, None]
        vis = torch.arange(L)[None, :] <= rows
        if chunk:
            vis = vis & (torch.arange(L)[None, :] >= rows // chunk * chunk)
        if sink:
            e = torch.exp(s - s.amax(-1, keepdim=True).clamp(min=0)) * vis
            p = e / (torch.exp(-s.amax(-1, keepdim=True).clamp(min=0)) + e.sum(-1, keepdim=True))
        else:
            p = torch.softmax(s.masked_fill(~vis, float("-inf")), -1)
        if all_groups:
            out[t0:t0 + n] = torch.einsum("hnl,lr->nhr", p, V.reshape(L, R))
        else:
            out[t0:t0 + n] = torch.einsum("hnl,lhv->nhv", p, V.repeat_interleave(rep, 1))
    return out


def sink_attn_mix(q, k_cache, v_cache, block_tables, cu, ctx_lens, talk, c: float, heads: int, kv_heads: int, dim: int,
                  vdim: int, scale: float, softcap: float, out, max_qlen: int = 0, num_decode: int = 0,
                  max_ctx: int = 0):
    """Sink attention, head mixing (``talk`` [heads, heads] or None) and the scale ``c`` in one op, written to
    ``out`` [T, heads * vdim]. ``max_qlen``, ``num_decode`` and ``max_ctx`` (an upper bound of every context length)
    only steer the choice of GPU kernels."""
    O = sink_attn(q, k_cache, v_cache, block_tables, cu, ctx_lens, heads, kv_heads, dim, vdim, scale, softcap,
                  talk is not None)
    return talk_mix(O, talk, c, heads, kv_heads, vdim, out=out)


def talk_mix(O, talk, c: float, heads: int, kv_heads: int, vdim: int, out=None, out_dtype=None):
    """y[t, h, :] = c * sum_h' talk[h, h'] O[t, h', group(h) part] (talk None: c * O). [T, heads * vdim]."""
    T = O.shape[0]
    rep = heads // kv_heads
    if talk is None:
        y = O.reshape(T, heads * vdim) * c
    else:
        Og = O.view(T, heads, kv_heads, vdim)
        grp = torch.arange(heads) // rep
        y = torch.einsum("hg,tghv->thv", talk.float(), Og[:, :, grp, :]).reshape(T, heads * vdim) * c
    if out is not None:
        out.copy_(y)
        return out
    return y.to(out_dtype)


# --------------------------------- blocks normed on the sublayer's output / depth average / bigram embedding / two maps
def embed_bigram(ids, positions, table, scale: float, bigram, mul_prev: int, mul_cur: int, prev, cu, ctx_lens,
                 state_slots, hist):
    """hist[0, t] = hist[1, t] = table[ids[t]] * scale + bigram[row], row = (previous * mul_prev + ids[t] * mul_cur)
    mod (len(bigram) - 1), or the table's last row at position 0. The token before a portion's first row is
    prev[slot] (int64 [slots]), which is set to the portion's last token here. hist fp32 [>= 2, T, W]."""
    buckets = bigram.shape[0] - 1
    slots = state_slots.tolist()
    idc = ids.clamp(0, table.shape[0] - 1)
    before = torch.zeros_like(idc)
    before[1:] = idc[:-1]
    for b, t0, n, p0 in _seq_rows(cu, ctx_lens):
        before[t0] = prev[slots[b]] if p0 > 0 else 0
        prev[slots[b]] = idc[t0 + n - 1]
    row = (before * mul_prev + idc * mul_cur) % buckets
    row = torch.where(positions == 0, torch.full_like(row, buckets), row)
    x = table[idc].float() * scale + bigram[row].float()
    hist[0].copy_(x)
    hist[1].copy_(x)


def resid_norm_add(hist, n: int, y, w, eps: float, dwa=None):
    """x = hist[n] (fp32 rows, in place) += rms_norm(y) * w. With ``dwa`` (fp32 [n + 1]) also hist[n + 1] =
    sum_{j <= n} dwa[j] hist[j], the sum taken over the updated x. Returns the rows the next reader takes: hist[n + 1]
    with dwa, else hist[n]."""
    yf = y.float()
    x = hist[n]
    x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * w.float())
    if dwa is None:
        return x
    hist[n + 1].copy_(torch.einsum("j,jtw->tw", dwa.float(), hist[:n + 1]))
    return hist[n + 1]


def gate_mul(y, src, col: int):
    """y[t, c] *= sigmoid(src[t, col + c]) in place (fp32 math)."""
    y.copy_((y.float() * torch.sigmoid(src[:, col:col + y.shape[1]].float())).to(y.dtype))
    return y


def qk_norm_cache(proj, off_q: int, off_k: int, off_v: int, qw, kw, eps: float, k_cache, v_cache, slots, heads: int,
                  kv_heads: int, maps: int, dim: int, vdim: int):
    """From the projection rows: queries [heads, maps, dim] and keys [kv_heads, maps, dim], each vector of ``dim``
    divided by its root mean square and multiplied by qw / kw (None: left as they are), values [kv_heads, vdim].
    Returns q fp32 [T, kv_heads * maps * rep * dim] ordered (key head, map, query head within the group): with the
    keys cached as kv_heads * maps heads, row-major (key head, map), query vector n reads key head n // rep. k / v go
    into the paged caches [blocks, block_size, kv_heads * maps * dim | kv_heads * vdim] at ``slots`` (< 0: skipped)."""
    T = proj.shape[0]
    rep = heads // kv_heads
    nq, nk, nv = heads * maps * dim, kv_heads * maps * dim, kv_heads * vdim

    def norm(x, w):
        if w is None:
            return x
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()
    q = norm(proj[:, off_q:off_q + nq].float().reshape(T, kv_heads, rep, maps, dim), qw)
    k = norm(proj[:, off_k:off_k + nk].float().reshape(T, kv_heads * maps, dim), kw)
    keep = slots >= 0
    k_cache.view(-1, nk)[slots[keep]] = k.reshape(T, nk)[keep].to(k_cache.dtype)
    v_cache.view(-1, nv)[slots[keep]] = proj[:, off_v:off_v + nv][keep].to(v_cache.dtype)
    return q.permute(0, 1, 3, 2, 4).reshape(T, nq).contiguous()


def diff_combine(O, lam: float, eps: float, mult: float, heads: int, kv_heads: int, vdim: int, out_dtype):
    """O fp32 [T, kv_heads * 2 * rep, vdim] ordered (key head, map, query head within the group) ->
    y[t, head] = mult * rms_div(O[map 0] - lam * O[map 1]) -> [T, heads * vdim] in ``out_dtype``."""
    T = O.shape[0]
    rep = heads // kv_heads
    Og = O.view(T, kv_heads, 2, rep, vdim)
    o = Og[:, :, 0] - lam * Og[:, :, 1]
    o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * mult
    return o.reshape(T, heads * vdim).to(out_dtype)



# ------------------- blocks normed on both sides / token input / windowed sigmoid attention with pooled blocks / SSD
def sandwich_add_norm(x, y, r, rb, wpost, eps: float, add, wnext, out_dtype):
    """x fp32 [T, W], in place: with ``y`` [T, W], x += rms_norm(y * sigmoid(r + rb)) * wpost (``r`` [T, W] gate
    logits and ``rb`` [W] their bias, or None for no gate; ``wpost`` fp32 [W]); with ``add`` (fp32 [T, W]) x += add;
    with ``wnext`` (fp32 [W]) returns rms_norm(x) * wnext in ``out_dtype``, else None."""
    if y is not None:
        yf = y.float()
        if r is not None:
            yf = yf * torch.sigmoid(r.float() + rb.float())
        x.add_(yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * wpost.float())
    if add is not None:
        x.add_(add)
    if wnext is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * wnext.float()).to(out_dtype)


def token_side_add(x, ids, table, col0: int, gate_w, proj_w, norm_w, eps: float, add, wnext, out_dtype):
    """x fp32 [T, W], in place: e = table[ids, col0 : col0 + d] (d = rows of gate_w); g = gelu_tanh(gate_w x) * e;
    y = proj_w g; x += rms_norm(y) * norm_w. Then ``add`` and ``wnext`` as in :func:`sandwich_add_norm`."""
    d = gate_w.shape[0]
    e = table[ids.clamp(0, table.shape[0] - 1), col0:col0 + d].float()
    g = torch.nn.functional.gelu(x @ gate_w.float().t(), approximate="tanh") * e
    y = g @ proj_w.float().t()
    x.add_(y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float())
    return sandwich_add_norm(x, None, None, None, None, eps, add, wnext, out_dtype)


def rope_pairs_cache(proj, off_q: int, off_k: int, off_v: int, cs, k_cache, v_cache, slots, heads: int,
                     kv_heads: int, dim: int, vdim: int):
    """From the projection rows: q and k with the neighbouring pairs (2i, 2i + 1), i < cs.shape[1], of every head
    turned by ``cs`` [T, dims / 2, 2] = (cos, sin) (None: no rotation), v as it is. Returns q fp32 [T, heads * dim];
    k / v go into the paged caches [blocks, block_size, kv_heads * dim | kv_heads * vdim] at ``slots`` (< 0: not
    cached)."""
    T = proj.shape[0]
    nq, nk, nv = heads * dim, kv_heads * dim, kv_heads * vdim
    q = proj[:, off_q:off_q + nq].float().reshape(T, heads, dim)
    k = proj[:, off_k:off_k + nk].float().reshape(T, kv_heads, dim)
    if cs is not None:
        q, k = _turn_neighbours(q, cs), _turn_neighbours(k, cs)
    keep = slots >= 0
    k_cache.view(-1, nk)[slots[keep]] = k.reshape(T, nk)[keep].to(k_cache.dtype)
    v_cache.view(-1, nv)[slots[keep]] = proj[:, off_v:off_v + nv][keep].to(v_cache.dtype)
    return q.reshape(T, nq).contiguous()


def pool_slot(block_tables, b: int, blk: int, pool: int, bs: int, per: int):
    """Row of the pooled caches that holds block ``blk`` of sequence ``b``: the page of the block's first position,
    and within it the block's rank among the blocks that start there."""
    p = blk * pool
    return int(block_tables[b, p // bs]) * per + (p % bs) // pool


def pool_update(k_cache, v_cache, kp_cache, vp_cache, block_tables, cu, ctx_lens, pool: int, max_qlen: int = 0):
    """Mean key and mean value (formed in fp32) of every block of ``pool`` positions whose last position the step has
    just written, from the cached rows of the block: kp_cache / vp_cache [blocks, ceil(block_size / pool), kv_heads *
    dim | vdim] in the pages' storage type, row :func:`pool_slot`. ``max_qlen`` (the step's longest portion) only sizes the GPU kernel's grid."""
    bs, per = k_cache.shape[1], kp_cache.shape[1]
    nk, nv = k_cache.shape[2], v_cache.shape[2]
    for b, _, n, p0 in _seq_rows(cu, ctx_lens):
        L = p0 + n
        for blk in range(p0 // pool, L // pool):  # p0 <= blk * pool + pool - 1 < L
            pos = torch.arange(blk * pool, blk * pool + pool)
            rows = block_tables[b, pos // bs].long() * bs + pos % bs
            s = pool_slot(block_tables, b, blk, pool, bs, per)
            kp_cache.view(-1, nk)[s] = k_cache.view(-1, nk)[rows].float().mean(0).to(kp_cache.dtype)
            vp_cache.view(-1, nv)[s] = v_cache.view(-1, nv)[rows].float().mean(0).to(vp_cache.dtype)


def pool_window_attn(q, k_cache, v_cache, kp_cache, vp_cache, block_tables, cu, ctx_lens, pb, heads: int,
                     kv_heads: int, dim: int, vdim: int, scale: float, window: int, pool: int, out_dtype,
                     max_qlen: int = 0, num_decode: int = 0, max_ctx: int = 0):
    """Sigmoid-weighted attention of every row over its sequence's cache: the row at position i adds sigmoid(q . k *
    scale + pb[head]) * v over the positions j with 0 <= i - j (< window when window > 0) and, when ``pool`` > 0, over
    the pooled rows of the blocks with blk * pool + pool - 1 <= i - window. q fp32 [T, heads * dim]; returns [T, heads
    * vdim] in ``out_dtype``. ``max_qlen``, ``num_decode`` and ``max_ctx`` only steer the GPU kernels."""
    T = q.shape[0]
    bs = k_cache.shape[1]
    rep = heads // kv_heads
    out = torch.zeros(T, heads, vdim, dtype=torch.float32)
    per = kp_cache.shape[1] if pool else 0
    for b, t0, n, p0 in _seq_rows(cu, ctx_lens):
        L = p0 + n
        blocks = block_tables[b, : -(-L // bs)].long()
        K = k_cache[blocks].reshape(-1, kv_heads, dim)[:L].float()
        V = v_cache[blocks].reshape(-1, kv_heads, vdim)[:L].float()
        nb = max(0, (L - window) // pool) if pool and window else 0
        if nb:
            rows = torch.tensor([pool_slot(block_tables, b, j, pool, bs, per) for j in range(nb)])
            K = torch.cat([K, kp_cache.view(-1, kv_heads, dim)[rows].float()], 0)
            V = torch.cat([V, vp_cache.view(-1, kv_heads, vdim)[rows].float()], 0)
        qq = q[t0:t0 + n].view(n, heads, dim).float()
        s = torch.einsum("nhd,lhd->hnl", qq, K.repeat_interleave(rep, 1)) * scale + pb.float()[:, None, None]
        i = (p0 + torch.arange(n))[:, None]
        j = torch.arange(L)[None, :]
        vis = (j <= i) & ((i - j < window) if window else torch.ones_like(j <= i))
        if nb:
            last = (torch.arange(nb) * pool + pool - 1)[None, :]
            vis = torch.cat([vis, last <= i - window], 1)
        p = torch.sigmoid(s) * vis
        out[t0:t0 + n] = torch.einsum("hnl,lhv->nhv", p, V.repeat_interleave(rep, 1))
    return out.reshape(T, heads * vdim).to(out_dtype)


def ssd_recurrence(x, Bm, Cm, dt, A_log, dt_bias, D, state, cu, ctx_lens, state_slots, heads: int, groups: int,
                   N: int, vdim: int):
    """Per head h (group g = h // (heads / groups)) over each sequence's rows: d = softplus(dt + dt_bias_h);
    S <- exp(-exp(A_log_h) d) S + d B_g x_h^T; y = S^T C_g + D_h x_h, S fp32 [slots, heads, N, vdim] carried in the
    sequence's slot (zero when the portion starts at position 0). x [T, heads * vdim], Bm / Cm [T, groups * N], dt [T,
    heads]. Returns fp32 [T, heads * vdim]."""
    T = x.shape[0]
    rep = heads // groups
    out = torch.zeros(T, heads * vdim, dtype=torch.float32)
    slots = state_slots.tolist()
    for b, t0, n, p0 in _seq_rows(cu, ctx_lens):
        S = state[slots[b]].clone() if p0 > 0 else torch.zeros(heads, N, vdim)
        xx = x[t0:t0 + n].float().view(n, heads, vdim)
        BB = Bm[t0:t0 + n].float().view(n, groups, N).repeat_interleave(rep, 1)
        CC = Cm[t0:t0 + n].float().view(n, groups, N).repeat_interleave(rep, 1)
        d = torch.nn.functional.softplus(dt[t0:t0 + n].float() + dt_bias.float(), threshold=20.0)
        a = torch.exp(-torch.exp(A_log.float()) * d)
        for j in range(n):
            S = a[j][:, None, None] * S + (d[j][:, None] * BB[j])[:, :, None] * xx[j][:, None, :]
            out[t0 + j] = (torch.einsum("hdv,hd->hv", S, CC[j]) + D.float()[:, None] * xx[j]).reshape(-1)
        state[slots[b]] = S
    return out
