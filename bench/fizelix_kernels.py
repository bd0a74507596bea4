"""Per-kernel rates of the Fizelix design beside the like kernel of the Llama family, at layer shapes of
bench/fizelix_compare.py, each at a prompt step (sequences of --seq tokens, --tokens in all) and a decode step
(--batch single tokens after --ctx cached ones). "of roofline" = the time the kernel's own roofline allows (the
larger of flops / 2.5 PFLOP/s and bytes / 8 TB/s) over the time measured. Prints one JSON object.

    python bench/fizelix_kernels.py [--size w2048] [--tokens 8192] [--seq 1024] [--batch 64] [--ctx 1024]
"""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "bench"))

from babotar_kernels import PEAK_TBS, PEAK_TFLOPS  # noqa: E402
from babotar_kernels import timed as timed_graph  # noqa: E402


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--size", default="w2048")
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=1000)
    a = ap.parse_args()
    from fizelix_compare import SIZES

    from llmss_amd import ops
    from llmss_amd.ops import hip as Hp

    s = SIZES[a.size]
    dev = torch.device("cuda", 0)
    bf = torch.bfloat16
    W = s["width"]
    H, G, D, win, pool = s["heads"], s["kv"], s["dim"], s["window"], s["pool"]
    SH, SV, N, SG = s["sheads"], s["svdim"], s["state"], s["groups"]
    E, top, EF, SF, F, side = s["experts"], s["top"], s["eff"], s["sff"], s["ff"], s["side"]
    gen = torch.Generator(device=dev).manual_seed(0)

    def rn(*shape, dt=bf, std=1.0):
        return (torch.randn(*shape, device=dev, generator=gen) * std).to(dt)

    def i32(x):
        return torch.tensor(x, dtype=torch.int32, device=dev)

    Hp.reserve_workspace(dev, 64 << 20)
    rows = []

    def add(name, phase, sec, flops=0.0, bytes_=0.0, like=None):
        ideal = max(flops / (PEAK_TFLOPS * 1e12), bytes_ / (PEAK_TBS * 1e12))
        rows.append(dict(kernel=name, phase=phase, us=round(sec * 1e6, 1), tflops=round(flops / sec / 1e12, 1),
                         tbs=round(bytes_ / sec / 1e12, 2), of_roofline=round(ideal / sec, 3), like=like))
        print(f"[kernels] {name} {phase}: {sec * 1e6:.1f} us, {ideal / sec:.3f} of roofline", file=sys.stderr, flush=True)

    bs = 16
    for phase in ("prompt", "decode"):
        def timed(fn, iters=10, warm=2, reps=8 if phase == "decode" else 1):
            return timed_graph(fn, iters=iters, warm=warm, reps=reps)

        if phase == "prompt":
            B, q, ctx = a.tokens // a.seq, a.seq, a.seq
        else:
            B, q, ctx = a.batch, 1, a.ctx + 1
        T = B * q
        cu = i32([i * q for i in range(B + 1)])
        cl = i32([ctx] * B)
        ss = i32(list(range(B)))
        nblk = -(-ctx // bs)
        bt = torch.arange(B * nblk, dtype=torch.int32, device=dev).view(B, nblk).contiguous()
        pos = (torch.arange(q, device=dev) + (ctx - q)).repeat(B)
        slots = (bt.long()[:, :, None] * bs + torch.arange(bs, device=dev)).view(B, -1)[:, ctx - q:ctx].reshape(-1).contiguous()
        # (query, key) pairs of the windowed, pooled mask
        vis = lambda p: min(p + 1, win) + max(0, (p - win + 1) // pool)
        pairs = B * sum(vis(p) for p in range(ctx - q, ctx))
        full = B * (q * (q + 1) // 2 + q * (ctx - q))

        # ---- the block's closing ops (Llama: residual add + RMS norm)
        x, y, r = rn(T, W, dt=torch.float32), rn(T, W), rn(T, W)
        f32 = lambda *sh: rn(*sh, dt=torch.float32)
        rb, wpost, wnext, add0 = f32(W), f32(W), f32(W), f32(T, W)
        t = timed(lambda: ops.sandwich_add_norm(x, y, r, rb, wpost, 1e-6, None, wnext, bf))
        add("sandwich_add_norm (gate, norm, scale, add, next norm)", phase, t, bytes_=T * W * (2 + 2 + 4 + 4 + 2))
        t = timed(lambda: ops.sandwich_add_norm(x, y, r, rb, wpost, 1e-6, add0, wnext, bf))
        add("sandwich_add_norm + embedding re-added", phase, t, bytes_=T * W * (2 + 2 + 4 + 4 + 4 + 2))
        xb, wb, rr = rn(T, W), rn(W), rn(T, W)
        t = timed(lambda: ops.add_norm(xb, wb, None, 1e-6, True, residual=rr))
        add("add_norm", phase, t, bytes_=T * W * 2 * 4, like="sandwich_add_norm")
        ids = torch.randint(0, s["vocab"], (T,), device=dev)
        table, sg, sp, sn = rn(s["vocab"], 4 * side), rn(side, W, std=W ** -0.5), rn(W, side), f32(W)
        t = timed(lambda: ops.token_side_add(x, ids, table, side, sg, sp, sn, 1e-6, None, wnext, bf))
        add("token_side_add (two small products, norm, add, next norm)", phase, t, flops=T * W * side * 4,
            bytes_=T * W * (4 + 4 + 2))
        # ---- attention: rotation + cache write, pooled means, windowed sigmoid attention
        nq, nk = H * D, G * D
        Np = nq + 2 * nk + W
        proj = rn(T, Np)
        kc, vc = rn(B * nblk, bs, nk), rn(B * nblk, bs, nk)
        per = -(-bs // pool)
        kp, vp = rn(B * nblk, per, nk), rn(B * nblk, per, nk)
        freqs = torch.tensor([10000.0 ** (-2.0 * i / (D // 2)) for i in range(D // 4)], device=dev)
        cs = ops.rope_angles(pos, freqs)
        t = timed(lambda: ops.rope_pairs_cache(proj, 0, nq, nq + nk, cs, kc, vc, slots, H, G, D, D))
        add("rope_pairs_cache", phase, t, bytes_=T * ((nq + 2 * nk) * 2 + nq * 4 + 2 * nk * 2))
        qf = ops.rope_pairs_cache(proj, 0, nq, nq + nk, cs, kc, vc, slots, H, G, D, D)
        t = timed(lambda: ops.pool_update(kc, vc, kp, vp, bt, cu, cl, pool, max_qlen=q))
        add("pool_update", phase, t, bytes_=B * (q // pool + 1) * 2 * nk * (pool * 2 + 2))
        pb = f32(H)
        f_att = lambda: ops.pool_window_attn(qf, kc, vc, kp, vp, bt, cu, cl, pb, H, G, D, D, D ** -0.5, win, pool, bf,
                                             max_qlen=q, max_ctx=ctx if phase == "decode" else 0)
        t = timed(f_att, iters=3, warm=1)
        seen_tok, seen_blk = min(ctx, win), max(0, (ctx - win) // pool)
        add("pool_window_attn", phase, t, flops=pairs * H * 4 * D,
            bytes_=(T * nq * 4 + B * 2 * nk * (seen_tok + seen_blk) * 2 + T * nq * 2) if phase == "decode" else 0)
        kc2, vc2 = rn(B * nblk, G, bs, D), rn(B * nblk, G, bs, D)
        if phase == "prompt":
            qkv = rn(T, (H + 2 * G) * D)
            t = timed(lambda: ops.attn_prefill(qkv, cu, q, H, G, D, D ** -0.5))
            add("attn_prefill (flash, full causal)", phase, t, flops=full * H * 4 * D, like="pool_window_attn")
        else:
            qd = rn(T, (H + 2 * G) * D)
            t = timed(lambda: ops.attn_decode(qd, kc2, vc2, bt, cl, H, G, D, D ** -0.5, ctx))
            add("attn_decode (split-K, all keys)", phase, t, bytes_=B * ctx * 2 * G * D * 2, like="pool_window_attn")
        # ---- state-space mixer
        inner, gn = SH * SV, SG * N
        C = inner + 2 * gn
        sproj = rn(T, 2 * inner + 2 * gn + SH, std=0.5)
        cw, cb, tail = rn(C, 4, std=0.5), rn(C, std=0.1), torch.zeros(B, 3, C, device=dev)
        f_conv = lambda: ops.causal_conv(sproj[:, inner:inner + C], cw, tail, cu, cl, ss, False, True, bf, bias=cb)
        t = timed(f_conv)
        add("causal_conv (4 taps, bias, SiLU, + tail)", phase, t, bytes_=T * C * 4)
        xbc = f_conv()
        A_log, dtb, Dk = f32(SH) * 0.5 - 0.5, f32(SH) * 0.5, f32(SH)
        state = torch.zeros(B, SH, N, SV, device=dev)
        f_rec = lambda: ops.ssd_recurrence(xbc[:, :inner], xbc[:, inner:inner + gn], xbc[:, inner + gn:],
                                           sproj[:, 2 * inner + 2 * gn:], A_log, dtb, Dk, state, cu, cl, ss, SH, SG, N, SV)
        t = timed(f_rec, iters=3, warm=1)
        add("ssd_recurrence", phase, t, flops=T * SH * N * SV * 4,
            bytes_=B * SH * N * SV * 8 + T * (C * 2 + inner * 4))
        yrec = f_rec()
        nw = rn(inner)
        t = timed(lambda: ops.gated_group_norm(yrec, sproj[:, :inner], nw, 1e-6, "silu", 1.0, out_dtype=bf, groups=1,
                                               gate_first=True))
        add("gated_group_norm (gate first)", phase, t, bytes_=T * inner * (4 + 2 + 2))
        # ---- experts: router, grouped gate / up with the score on the input, down
        h = rn(T, W)
        rw = rn(E, W, std=W ** -0.5)
        t = timed(lambda: ops.moe_router(h, rw, None, top, False))
        add("moe_router", phase, t, flops=T * W * E * 2, bytes_=T * W * 2)
        idx, wts = ops.moe_router(h, rw, None, top, False)
        eg, eu, ed = rn(E, EF, W, std=W ** -0.5), rn(E, EF, W, std=W ** -0.5), rn(E, W, EF, std=EF ** -0.5)
        t = timed(lambda: ops.moe_experts(h, idx, wts, eg, eu, ed, 0.0, 1.702, shared=None, combine=False, act="silu",
                                          weight_input=True), iters=5)
        touched = min(E, T * top)
        add("experts (group + grouped gate/up + down)", phase, t, flops=T * top * W * EF * 6,
            bytes_=touched * 3 * W * EF * 2)
        # ---- dense feed-forward with the gate of the residual riding in the first GEMM; Llama's fused one
        gu_w, dn_w = rn(2 * F + W, W, std=W ** -0.5), rn(W, F, std=F ** -0.5)
        t = timed(lambda: ops.linear_f(ops.glu_act(ops.linear_f(h, gu_w, bf), F, "silu"), dn_w, bf))
        add("feed-forward (gate | up | residual gate GEMM, glu_act, down GEMM)", phase, t,
            flops=T * W * (3 * F + W) * 2, bytes_=(3 * F + W) * W * 2)
        g_w, u_w, d_w = rn(F, W, std=W ** -0.5), rn(F, W, std=W ** -0.5), rn(W, F, std=F ** -0.5)
        gu_i = ops.glu_interleave(g_w, u_w).contiguous()
        t = timed(lambda: ops.linear(ops.linear(h, gu_i, None, "none", True), d_w))
        add("gated MLP (fused epilogue)", phase, t, flops=T * W * F * 6, bytes_=3 * W * F * 2, like="feed-forward")
        # ---- the mixers' input GEMMs
        pw = rn(-(-Np // 8) * 8, W, std=W ** -0.5)
        t = timed(lambda: ops.linear_f(h, pw, bf))
        add("attention input GEMM (q | k | v | gate)", phase, t, flops=T * W * Np * 2, bytes_=W * Np * 2)
        Ns = -(-(2 * inner + 2 * gn + SH + W) // 8) * 8
        pw2 = rn(Ns, W, std=W ** -0.5)
        t = timed(lambda: ops.linear_f(h, pw2, bf))
        add("state-space input GEMM (z | x | B | C | dt | gate)", phase, t, flops=T * W * Ns * 2, bytes_=W * Ns * 2)
    print(json.dumps(dict(size=a.size, shape=s, tokens=a.tokens, seq=a.seq, batch=a.batch, ctx=a.ctx, kernels=rows)))


if __name__ == "__main__":
    main()
