"""Per-kernel rates of the Lamisun design beside the like kernel of the Llama family, at layer shapes of
bench/lamisun_compare.py, each at a prompt step (sequences of --seq tokens, --tokens in all) and a decode step
(--batch single tokens after --ctx cached ones). "of roofline" = the time the kernel's own roofline allows (the
larger of flops / 2.5 PFLOP/s and bytes / 8 TB/s) over the time measured. Prints one JSON object.

    python bench/lamisun_kernels.py [--size w2048] [--tokens 8192] [--seq 1024] [--batch 64] [--ctx 1024]
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
    ap.add_argument("--depth", type=int, default=4, help="earlier results the depth average of the timed layer reads")
    a = ap.parse_args()
    from lamisun_compare import SIZES

    from llmss_amd import ops
    from llmss_amd.ops import hip as Hp

    s = SIZES[a.size]
    dev = torch.device("cuda", 0)
    bf = torch.bfloat16
    W, F = s["width"], s["ff"]
    LH, LD, LR, LV, R = s["lheads"], s["ldim"], s["lrot"], s["lvdim"], s["rank"]
    H, G, D, DV, chunk = s["heads"], s["kv"], s["dim"], s["vdim"], s["chunk"]
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
        # a decode step's kernels take microseconds: eight calls per graph, so that the replay's floor is shared
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
        pairs = B * (q * (q + 1) // 2 + q * (ctx - q))  # (query, key) pairs a causal step touches
        n_ch = sum(min(p % chunk, p) + 1 for p in range(ctx - q, ctx)) * B if chunk else pairs  # inside the chunks

        # ---- embedding: token row + bigram row into two result slots
        ids = torch.randint(0, s["vocab"], (T,), device=dev)
        table, big = rn(s["vocab"], W), rn(s["buckets"] + 1, W)
        prev = torch.zeros(B, dtype=torch.int64, device=dev)
        n = a.depth
        hist = rn(n + 2, T, W, dt=torch.float32)
        t = timed(lambda: ops.embed_bigram(ids, pos, table, 1.0, big, 1000003, 7919, prev, cu, cl, ss, hist))
        add("embed_bigram", phase, t, bytes_=T * W * (2 + 2 + 8))
        # ---- residual: x += norm(y) w, and the depth average over n + 1 results (Llama: residual add + RMS norm)
        y, w = rn(T, W), rn(W)
        dwa = rn(n + 1, dt=torch.float32)
        t = timed(lambda: ops.resid_norm_add(hist, n, y, w, 1e-6, None))
        add("resid_norm_add", phase, t, bytes_=T * W * (2 * 2 + 4 + 4))
        t = timed(lambda: ops.resid_norm_add(hist, n, y, w, 1e-6, dwa))
        add(f"resid_norm_add + depth average of {n + 1}", phase, t, bytes_=T * W * (2 * 2 + 4 + 4 + 4 * n + 4))
        r, xb = rn(T, W), rn(T, W)
        t = timed(lambda: ops.add_norm(xb, w, None, 1e-6, True, residual=r))
        add("add_norm", phase, t, bytes_=T * W * 2 * 4, like="resid_norm_add")
        # ---- input convolution over the fp32 residual (no Llama counterpart)
        cw, tail = rn(W, 4), torch.zeros(B, 3, W, device=dev)
        t = timed(lambda: ops.causal_conv(hist[1], cw, tail, cu, cl, ss, True, False, bf))
        add("causal_conv (4 taps, + tail)", phase, t, bytes_=T * W * (4 + 2))
        # ---- latent attention
        Rt = R + LR
        nq = LH * (LD + LR)
        Np = -(-(nq + Rt + LH * LV) // 8) * 8
        qc = rn(T, Np)
        cache = rn(B * nblk, bs, Rt)
        uk_t, uv, nw = rn(LH, R, LD, std=R ** -0.5), rn(LH * LV, R, std=R ** -0.5), rn(R)
        freqs = torch.tensor([10000.0 ** (-2.0 * i / LR) for i in range(LR // 2)], device=dev)
        t = timed(lambda: ops.rope_angles(pos, freqs))
        add("rope_angles", phase, t, bytes_=T * LR * 4)
        cs = ops.rope_angles(pos, freqs)
        qdt = ops.latent_qa_dtype(cache)
        t = timed(lambda: ops.head_absorb(qc, uk_t, qdt, extra=LR))
        add("head_absorb", phase, t, flops=T * LH * LD * R * 2, bytes_=T * LH * (LD * 2 + R * 2))
        qa = ops.head_absorb(qc, uk_t, qdt, extra=LR)
        t = timed(lambda: ops.latent_norm_cache(qc, nq, R, nw, 1e-6, cache, slots, LR, cs, qa, 0, LD))
        add("latent_norm_cache (norm, rotation, cache write)", phase, t, bytes_=T * (Rt * 4 + LH * LR * 4))
        single = phase == "decode"
        f_lat = lambda: ops.latent_attn(qa, cache, bt, cu, cl, 0, 0.07, max_qlen=q, max_ctx=ctx if single else 0)
        t = timed(f_lat, iters=3, warm=1)
        add("latent_attn (row of rank + rotated part)", phase, t, flops=pairs * LH * 4 * Rt,
            bytes_=(B * ctx * Rt * 2 + T * LH * Rt * 4) if single else 0)
        o = f_lat()
        t = timed(lambda: ops.head_expand(o, uv, bf))
        add("head_expand", phase, t, flops=T * LH * LV * R * 2, bytes_=T * LH * (Rt * 2 + LV * 2))
        yv = ops.head_expand(o, uv, bf)
        t = timed(lambda: ops.gate_mul(yv, qc, nq + Rt))
        add("gate_mul", phase, t, bytes_=T * LH * LV * 2 * 3)
        # ---- two-map attention
        mq, mk, mv = H * 2 * D, G * 2 * D, G * DV
        proj = rn(T, mq + mk + mv)
        kc, vc = rn(B * nblk, bs, mk), rn(B * nblk, bs, mv)
        qw, kw = rn(D), rn(D)
        t = timed(lambda: ops.qk_norm_cache(proj, 0, mq, mq + mk, qw, kw, 1e-6, kc, vc, slots, H, G, 2, D, DV))
        add("qk_norm_cache", phase, t, bytes_=T * ((mq + mk + mv) * 2 + mq * 4 + (mk + mv) * 2))
        qf = ops.qk_norm_cache(proj, 0, mq, mq + mk, qw, kw, 1e-6, kc, vc, slots, H, G, 2, D, DV)
        vis = (ctx - 1) % chunk + 1 if chunk else ctx  # keys the last position sees
        f_two = lambda: ops.sink_attn(qf, kc, vc, bt, cu, cl, 2 * H, 2 * G, D, DV, D ** -0.5, 0.0, False, max_qlen=q,
                                      sink=False, chunk=chunk, vshare=2, precise=True)
        t = timed(f_two, iters=3, warm=1)
        add("two-map attention (sink_attn, 32-bit weights)", phase, t, flops=n_ch * 2 * H * 2 * (D + DV),
            bytes_=(T * mq * 4 + B * vis * (mk + mv) * 2 + T * 2 * H * DV * 4) if single else 0)
        f_two16 = lambda: ops.sink_attn(qf, kc, vc, bt, cu, cl, 2 * H, 2 * G, D, DV, D ** -0.5, 0.0, False, max_qlen=q,
                                        sink=False, chunk=chunk, vshare=2, precise=False)
        t = timed(f_two16, iters=3, warm=1)
        add("two-map attention (sink_attn, bf16 weights)", phase, t, flops=n_ch * 2 * H * 2 * (D + DV),
            bytes_=(T * mq * 4 + B * vis * (mk + mv) * 2 + T * 2 * H * DV * 4) if single else 0)
        O = f_two()
        t = timed(lambda: ops.diff_combine(O, 0.4, 1e-6, 0.7, H, G, DV, bf))
        add("diff_combine", phase, t, bytes_=T * H * DV * (8 + 2))
        # Llama's: flash prefill / split-K decode, heads of 2 D
        D2 = 2 * D
        kc2, vc2 = rn(B * nblk, G, bs, D2), rn(B * nblk, G, bs, D2)
        if phase == "prompt":
            qkv = rn(T, (H + 2 * G) * D2)
            t = timed(lambda: ops.attn_prefill(qkv, cu, q, H, G, D2, D2 ** -0.5))
            add("attn_prefill (flash)", phase, t, flops=pairs * H * 4 * D2, like="two-map attention / latent_attn")
        else:
            qd = rn(T, (H + 2 * G) * D2)
            t = timed(lambda: ops.attn_decode(qd, kc2, vc2, bt, cl, H, G, D2, D2 ** -0.5, ctx))
            add("attn_decode (split-K)", phase, t, bytes_=B * ctx * 2 * G * D2 * 2, like="two-map attention / latent_attn")
        # ---- feed-forward: up GEMM + xIELU + down GEMM (Llama: gated, activation in the GEMM epilogue)
        h = rn(T, W)
        up_w, dn_w = rn(F, W, std=W ** -0.5), rn(W, F, std=F ** -0.5)
        u = ops.linear_f(h, up_w, bf)
        t = timed(lambda: ops.act_fn(u, "xielu", (0.8, 1.2)))
        add("act_fn (xIELU)", phase, t, bytes_=T * F * 4)
        t = timed(lambda: ops.linear_f(ops.act_fn(ops.linear_f(h, up_w, bf), "xielu", (0.8, 1.2)), dn_w, bf))
        add("feed-forward (2 GEMMs + act_fn)", phase, t, flops=T * W * F * 4, bytes_=2 * W * F * 2)
        Fd = F * 2 // 3 // 64 * 64
        g_w, u_w, d_w = rn(Fd, W, std=W ** -0.5), rn(Fd, W, std=W ** -0.5), rn(W, Fd, std=Fd ** -0.5)
        gu_i = ops.glu_interleave(g_w, u_w).contiguous()
        t = timed(lambda: ops.linear(ops.linear(h, gu_i, None, "none", True), d_w))
        add("gated MLP (fused epilogue)", phase, t, flops=T * W * Fd * 6, bytes_=3 * W * Fd * 2, like="feed-forward")
        # ---- the mixers' input and output GEMMs
        pw = rn(Np, W, std=W ** -0.5)
        t = timed(lambda: ops.linear_f(h, pw, bf))
        add("latent input GEMM (q | latent | gate)", phase, t, flops=T * W * Np * 2, bytes_=W * Np * 2)
        pw2 = rn(mq + mk + mv, W, std=W ** -0.5)
        t = timed(lambda: ops.linear_f(h, pw2, bf))
        add("two-map input GEMM (q | k | v)", phase, t, flops=T * W * (mq + mk + mv) * 2, bytes_=W * (mq + mk + mv) * 2)
    print(json.dumps(dict(size=a.size, shape=s, tokens=a.tokens, seq=a.seq, batch=a.batch, ctx=a.ctx, kernels=rows)))


if __name__ == "__main__":
    main()
