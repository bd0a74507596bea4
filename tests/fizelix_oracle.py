"""Plain float64 definition of the Fizelix design: one function per mechanism, whole sequences, no cache, no batching.

It takes the config as the dictionary a ``config.json`` holds and the weights as a dictionary of checkpoint names, and
shares no code with the framework's model path. Slow on purpose: every loop is the equation it stands for.
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rotate_pairs(x, positions, dims, base):
    """x [T, heads, dim]: the pairs (2i, 2i + 1), i < dims / 2, turned by position * base^(-2i / dims)."""
    out = x.clone()
    for i in range(dims // 2):
        a = positions.to(F64) * base ** (-2.0 * i / dims)
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def window_pool_attention(q, k, v, pb, scale, size, pool):
    """q [T, H, dim], k [T, G, dim], v [T, G, vdim] (k already rotated). Position i sees the tokens j with
    0 <= i - j < size and one mean key / value for every block of ``pool`` tokens that ends at or before i - size.
    Weight of whatever it sees: sigmoid(score * scale + pb[h]); weights are not normalised."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=F64)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            keys = [k[j, g] for j in range(max(0, i - size + 1) if size else 0, i + 1)]
            vals = [v[j, g] for j in range(max(0, i - size + 1) if size else 0, i + 1)]
            b = 0
            while size and pool and b * pool + pool - 1 <= i - size:
                keys.append(k[b * pool:(b + 1) * pool, g].mean(0))
                vals.append(v[b * pool:(b + 1) * pool, g].mean(0))
                b += 1
            wgt = torch.sigmoid(torch.stack(keys) @ q[i, h] * scale + pb[h])
            out[i, h] = wgt @ torch.stack(vals)
    return out


def attention_mixer(w, p, m, h):
    T = h.shape[0]
    H, G, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[p + "q"].T).view(T, H, dim)
    k = (h @ w[p + "k"].T).view(T, G, dim)
    v = (h @ w[p + "v"].T).view(T, G, vdim)
    pos = torch.arange(T)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        q = rotate_pairs(q, pos, rot["dims"], rot["base"])
        k = rotate_pairs(k, pos, rot["dims"], rot["base"])
    mask = m.get("mask") or {}
    o = window_pool_attention(q, k, v, w[p + "pb"], m["scale"], mask.get("size", 0), mask.get("pool", 0))
    return o.reshape(T, H * vdim) @ w[p + "o"].T


def causal_conv(x, cw, cb):
    """x [T, C], cw [C, taps] (last column: the current token), zeros before the start."""
    T, C = x.shape
    taps = cw.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        acc = cb.clone()
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                acc = acc + cw[:, j] * x[s]
        out[t] = acc
    return out


def ssd_scan(x, B, C, dt, A_log, D, heads, groups):
    """x [T, heads, vdim], B / C [T, groups, N], dt [T, heads] (after softplus). S_t = exp(-exp(A_log) dt) S_(t-1) +
    dt B_t x_t^T ; y_t = S_t^T C_t + D x_t."""
    T, _, vdim = x.shape
    N = B.shape[2]
    y = torch.zeros(T, heads, vdim, dtype=F64)
    for h in range(heads):
        g = h // (heads // groups)
        S = torch.zeros(N, vdim, dtype=F64)
        for t in range(T):
            S = torch.exp(-torch.exp(A_log[h]) * dt[t, h]) * S + dt[t, h] * torch.outer(B[t, g], x[t, h])
            y[t, h] = S.T @ C[t, g] + D[h] * x[t, h]
    return y


def mamba2_mixer(w, p, m, h, eps):
    T = h.shape[0]
    heads, vdim, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * vdim
    proj = h @ w[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, w[p + "conv"], w[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, heads, vdim)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + "dt_bias"])
    y = ssd_scan(x, B, C, dt, w[p + "A_log"], w[p + "D"], heads, G).reshape(T, inner)
    y = y * silu(z)
    ng = m["norm_groups"]
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w[p + "norm"]
    return y @ w[p + "o"].T


def gated_mlp(w, p, h):
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def moe(w, p, f, h):
    """Sigmoid scores, the ``top`` largest chosen, the score multiplies the expert's INPUT; a shared expert is added."""
    s = torch.sigmoid(h @ w[p + "router"].T)
    top = f["router"]["top"]
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=F64)
    for t in range(h.shape[0]):
        order = sorted(range(s.shape[1]), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            out[t] += gated_mlp(w, f"{p}e{e}.", (s[t, e] * h[t])[None])[0]
    if f.get("shared"):
        out = out + gated_mlp(w, p + "shared.", h)
    return out


def gated_post_norm(y, h, rg, rgb, normb, ls, eps):
    """What a sublayer adds to the residual: its result y times sigmoid(rg h + rgb), RMS-normed with weight normb,
    times the layer scale ls."""
    return rms(y * torch.sigmoid(h @ rg.T + rgb), eps) * normb * ls


def token_side(x, e, gate, proj, norm, eps):
    """What the token input adds: e [T, d] the layer's slice of the token table's rows."""
    return rms((gelu_tanh(x @ gate.T) * e) @ proj.T, eps) * norm


def layer_runs(cfg):
    """Layer indices in the order they run: layers start .. stop - 1 ``times`` times in a row. Second item: whether
    the embedding output is added right before this run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop or loop.get("times", 1) <= 1:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    runs = [(i, False) for i in range(a)]
    for r in range(times):
        runs += [(i, r > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg, weights, tokens, taps=None):
    """Logits [T, vocab] of one sequence; ``taps``: a list that receives the residual after every layer run."""
    w = {k: v.to(F64) if v.is_floating_point() else v for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x0 = w["embed"][tok] * cfg["embedding"]["scale"]
    x = x0.clone()
    side = cfg.get("token_side")
    for i, again in layer_runs(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if again:
            x = x + x0
        h = rms(x, eps) * w[p + "norm1"]
        if L["type"] == "attention":
            y = attention_mixer(w, p + "mix.", L["mixer"], h)
        elif L["type"] == "mamba2":
            y = mamba2_mixer(w, p + "mix.", L["mixer"], h, eps)
        else:
            raise ValueError(L["type"])
        x = x + gated_post_norm(y, h, w[p + "rg1"], w[p + "rg1.b"], w[p + "norm1b"], w[p + "ls1"], eps)
        if L.get("mlp"):
            h = rms(x, eps) * w[p + "norm2"]
            f = L["mlp"]
            y = gated_mlp(w, p + "mlp.", h) if f["kind"] == "dense" else moe(w, p + "mlp.", f, h)
            x = x + gated_post_norm(y, h, w[p + "rg2"], w[p + "rg2.b"], w[p + "norm2b"], w[p + "ls2"], eps)
        if side:
            d = side["dim"]
            e = w["side.embed"][tok][:, i * d:(i + 1) * d]
            x = x + token_side(x, e, w[p + "side.gate"], w[p + "side.proj"], w[p + "side.norm"], eps)
        if taps is not None:
            taps.append(x.clone())
    h = rms(x, eps) * w["final.norm"]
    return (h @ w["head"].T) * cfg.get("logit_scale", 1.0)


def greedy(cfg, weights, prompt, n):
    """n tokens generated greedily (the whole sequence recomputed for every token)."""
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]
