"""Plain definition of the Lamisun design in float64: one function per mechanism, whole sequences, no cache, no
batching, nothing shared with the product path. ``forward`` takes the raw config dictionary and a name -> tensor
dictionary under the checkpoint's names and returns the logits of every position and the residual stream after
every layer."""
import math

import torch

F64 = torch.float64


def rms_div(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def xielu(z, p, q):
    """Quadratic above zero, saturating exponential below; p and q are the raw (pre-softplus) numbers."""
    ap, aq = softplus(float(p)), 0.5 + softplus(float(q))
    pos = ap * z * z + 0.5 * z
    neg = aq * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def embed(tokens, table, bigram, scale, buckets, mul_prev, mul_cur):
    """Token row times ``scale`` plus a hashed row of the (previous, current) pair; the first token takes the
    table's last row."""
    x = torch.zeros(len(tokens), table.shape[1], dtype=F64)
    for t, tok in enumerate(tokens):
        row = buckets if t == 0 else (int(tokens[t - 1]) * mul_prev + int(tok) * mul_cur) % buckets
        x[t] = table[int(tok)] * scale + bigram[row]
    return x


def causal_conv(h, w):
    """h [T, C], w [C, taps]; column taps - 1 multiplies the current row, column 0 the row taps - 1 back."""
    T, C = h.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                out[t] += w[:, j] * h[s]
    return out


def rotate_pairs(x, base, dims):
    """x [T, ..., n]: the first ``dims`` numbers of the last axis turn, neighbours (2i, 2i + 1) forming a pair that
    turns by position * base^(-2i / dims)."""
    T = x.shape[0]
    out = x.clone()
    for i in range(dims // 2):
        ang = torch.arange(T, dtype=F64) * base ** (-2.0 * i / dims)
        c = torch.cos(ang).view(T, *([1] * (x.dim() - 2)))
        s = torch.sin(ang).view(T, *([1] * (x.dim() - 2)))
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def visible(T, chunk=0):
    """[T, T] booleans: key j is seen from position i when j <= i and, with ``chunk`` > 0, both lie in the same
    block of ``chunk`` positions counted from 0."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = j <= i
    if chunk:
        vis = vis & (i // chunk == j // chunk)
    return vis


def softmax_rows(s, vis):
    s = s.masked_fill(~vis, float("-inf"))
    e = torch.exp(s - s.amax(-1, keepdim=True))
    return e / e.sum(-1, keepdim=True)


def latent_heads(q, down, norm_w, uk, uv, H, d, r, dv, R, base, scale, eps, dims=None):
    """q [T, H * (d + r)] (per head: d plain numbers, then r of which the first ``dims`` turn with the position),
    down [T, R + r] (the latent before its norm, then one such key part for all heads). Returns the heads' outputs
    [T, H * dv]."""
    T = q.shape[0]
    dims = r if dims is None else dims
    q = q.view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_pairs(q[..., d:], base, dims)
    c = rms_div(down[:, :R], eps) * norm_w
    k_rot = rotate_pairs(down[:, R:], base, dims)
    k_plain = (c @ uk.T).view(T, H, d)
    v = (c @ uv.T).view(T, H, dv)
    vis = visible(T)
    heads = []
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * scale
        heads.append(softmax_rows(s, vis) @ v[:, a])
    return torch.cat(heads, -1)


def latent_attention(h, m, w, eps):
    """h [T, W]; m the mixer's config; w maps short names (q, dkv, dkv.norm, uk, uv, g, o) to tensors."""
    H, d, r, dv, R = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    o = latent_heads(h @ w["q"].T, h @ w["dkv"].T, w["dkv.norm"], w["uk"], w["uv"], H, d, r, dv, R,
                     float(m["rot"]["base"]), float(m["scale"]), eps, int(m["rot"]["dims"]))
    return (o * torch.sigmoid(h @ w["g"].T)) @ w["o"].T


def two_map_heads(q, k, v, scale, lam, mult, chunk, eps):
    """q [T, H, 2, d], k [T, G, 2, d] (already normed), v [T, G, dv]: per head two softmax maps over the same values,
    o = map 0 - lam * map 1, divided by its root mean square, times mult. Returns [T, H * dv]."""
    T, H = q.shape[0], q.shape[1]
    G = k.shape[1]
    vis = visible(T, chunk)
    heads = []
    for a in range(H):
        g = a // (H // G)
        maps = [softmax_rows((q[:, a, n] @ k[:, g, n].T) * scale, vis) @ v[:, g] for n in range(2)]
        heads.append(rms_div(maps[0] - lam * maps[1], eps) * mult)
    return torch.cat(heads, -1)


def second_map_weight(lq1, lk1, lq2, lk2, diff):
    return math.exp(float((lq1 * lk1).sum())) - math.exp(float((lq2 * lk2).sum())) + diff


def diff_attention(h, m, w, eps):
    """Two softmax maps per head over the same values, the second subtracted with one learned weight per layer;
    h [T, W]; w maps short names (q, k, v, q.norm, k.norm, lq1, lk1, lq2, lk2, o) to tensors."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    diff = float(m["diff"])
    q = rms_div((h @ w["q"].T).view(T, H, 2, d), eps) * w["q.norm"]
    k = rms_div((h @ w["k"].T).view(T, G, 2, d), eps) * w["k.norm"]
    v = (h @ w["v"].T).view(T, G, dv)
    lam = second_map_weight(w["lq1"], w["lk1"], w["lq2"], w["lk2"], diff)
    o = two_map_heads(q, k, v, float(m["scale"]), lam, 1.0 - diff, int((m.get("mask") or {}).get("size") or 0), eps)
    return o @ w["o"].T


def feed_forward(h, w):
    return xielu(h @ w["up"].T, w["act"][0], w["act"][1]) @ w["down"].T


MIXERS = {"latent_attention": latent_attention, "attention": diff_attention}


def forward(cfg, sd, tokens):
    """(logits [T, vocab], residual after every layer [layers, T, W]) in float64."""
    sd = {k: v.to(F64) for k, v in sd.items()}
    eps = float(cfg["norm"]["eps"])
    bg = cfg["embedding"]["bigram"]
    x = embed(tokens, sd["embed"], sd["bigram"], float(cfg["embedding"]["scale"]), int(bg["buckets"]),
              int(bg["mul_prev"]), int(bg["mul_cur"]))
    results = [x]  # what every layer produced, the embedding first
    after = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."

        def part(pre):
            return {k[len(p + pre):]: v for k, v in sd.items() if k.startswith(p + pre)}
        h = x + causal_conv(x, sd[p + "canon1"])
        x = x + rms_div(MIXERS[L["type"]](h, L["mixer"], part("mix."), eps), eps) * sd[p + "norm1"]
        if L.get("mlp") is not None:
            h = x + causal_conv(x, sd[p + "canon2"])
            x = x + rms_div(feed_forward(h, part("mlp.")), eps) * sd[p + "norm2"]
        results.append(x)
        x = sum(sd[p + "dwa"][j] * results[j] for j in range(i + 2))
        after.append(x)
    y = rms_div(x, eps) * sd["final.norm"]
    return y @ sd["head"].T, torch.stack(after)


def greedy(cfg, sd, prompt, n):
    """The n tokens greedy decoding appends to the prompt (the whole sequence is recomputed for every token)."""
    seq, out = list(prompt), []
    for _ in range(n):
        tok = int(forward(cfg, sd, seq)[0][-1].argmax())
        out.append(tok)
        seq.append(tok)
    return out
