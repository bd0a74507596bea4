"""Per-kernel rates of the Babotar design beside the like kernel of the Llama family, at layer shapes of
bench/babotar_compare.py, each at a prompt step (sequences of --seq tokens, --tokens in all) and a decode step
(--batch single tokens after --ctx cached ones). "of roofline" = the time the kernel's own roofline allows (the
larger of flops / 2.5 PFLOP/s and bytes / 8 TB/s) over the time measured. Prints one JSON object.

    python bench/babotar_kernels.py [--size w2048] [--tokens 8192] [--seq 1024] [--batch 64] [--ctx 1024]
"""
import argparse
import json
import os
import sys

import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "bench"))

PEAK_TFLOPS, PEAK_TBS = 2500.0, 8.0


def timed(fn, iters=10, warm=2, reps=1):
    """Device seconds per call: the call is captured into a HIP graph and the graph replayed, so the host-side
    launcher (argument checks, allocations) is not part of the time. ``reps`` > 1 captures that many calls back to
    back, as a decode graph holds a kernel among many others: the floor of replaying a graph is then shared."""
    for _ in range(warm):
        fn()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    with torch.cuda.graph(g):
        for _ in range(reps):
            fn()
    g.replay()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        g.replay()
    b.record()
    b.synchronize()
    return a.elapsed_time(b) / (iters * reps) * 1e-3


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--size", default="w2048")
    ap.add_argument("--tokens", type=int, default=8192)
    ap.add_argument("--seq", type=int, default=1024)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--ctx", type=int, default=1024)
    a = ap.parse_args()
    from babotar_compare import SIZES

    from llmss_amd import ops
    from llmss_amd.ops import hip as Hp

    s = SIZES[a.size]
    dev = torch.device("cuda", 0)
    bf = torch.bfloat16
    W, H, G, D, rot = s["width"], s["heads"], s["kv"], s["dim"], s["rot"]
    dH, dG, dD, dV = s["dheads"], s["dkv"], s["ddim"], s["dvdim"]
    lH, lD, lV, F = s["lheads"], s["ldim"], s["lvdim"], s["ff"]
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

        # ---- streams: write-back + normed read (Llama: residual add + RMS norm)
        x = rn(2, T, W, dt=torch.float32)
        y, w = rn(T, W), rn(W)
        mix, outw, inw = rn(2, 2, dt=torch.float32), rn(2, dt=torch.float32), rn(2, dt=torch.float32)
        t = timed(lambda: ops.stream_add_norm(x, y, mix, outw, 1.0, inw, w, 1e-6, False, bf))
        add("stream_add_norm (2 streams)", phase, t, bytes_=T * W * (4 * 4 + 2 + 2))
        r, xb = rn(T, W), rn(T, W)
        t = timed(lambda: ops.add_norm(xb, w, None, 1e-6, True, residual=r))
        add("add_norm", phase, t, bytes_=T * W * 2 * 4, like="stream_add_norm")
        # ---- input convolution (no Llama counterpart)
        hf = rn(T, W, dt=torch.float32)
        cw, tail = rn(W, 4), torch.zeros(B, 3, W, device=dev)
        t = timed(lambda: ops.causal_conv(hf, cw, tail, cu, cl, ss, True, False, bf))
        add("causal_conv (4 taps, + tail)", phase, t, bytes_=T * W * (4 + 2))
        # ---- rotation + bias + cache write (Llama: rope_cache)
        nq, nk, nv = H * D, G * D, G * D
        proj = rn(T, nq + nk + nv)
        bias = rn(nq + nk + nv)
        kc, vc = rn(B * nblk, bs, nk), rn(B * nblk, bs, nv)
        tab = ops.rope_angle_table(8192, rot, 10000.0, (4.0, 4096.0, 16.0, 2.0)).to(dev)
        t = timed(lambda: ops.rope_bias_cache(proj, 0, nq, nq + nk, bias, pos, tab, rot, kc, vc, slots, H, G, D, D))
        add("rope_bias_cache", phase, t, bytes_=T * ((nq + nk + nv) * 2 + nq * 4 + (nk + nv) * 2))
        # ---- attention
        qf = rn(T, nq, dt=torch.float32)
        talk = rn(H, H, dt=torch.float32)
        fl = pairs * H * 2 * (D + G * D)  # scores + weighted sums over all G value groups
        by = (T * nq * 4 + B * ctx * (nk + nv) * 2 + T * H * G * D * 4) if phase == "decode" else 0
        f_attn = lambda: ops.sink_attn(qf, kc, vc, bt, cu, cl, H, G, D, D, D ** -0.5, 30.0, True, max_qlen=q)
        t = timed(f_attn, iters=3, warm=1)
        add("sink_attn (all value groups)", phase, t, flops=fl, bytes_=by)
        O = f_attn()
        both = torch.empty(T, H * D + dH * dV, dtype=bf, device=dev)
        t = timed(lambda: ops.talk_mix(O, talk, 1.0, H, G, D, out=both[:, :H * D]))
        add("talk_mix", phase, t, flops=T * H * H * D * 2, bytes_=T * (H * G * D * 4 + H * D * 2))
        # Llama's: flash prefill / split-K decode over a [blocks, kv heads, block, D] cache
        kc2, vc2 = rn(B * nblk, G, bs, D), rn(B * nblk, G, bs, D)
        if phase == "prompt":
            qkv = rn(T, (H + 2 * G) * D)
            t = timed(lambda: ops.attn_prefill(qkv, cu, q, H, G, D, D ** -0.5))
            add("attn_prefill (flash)", phase, t, flops=pairs * H * 4 * D, like="sink_attn")
        else:
            qd = rn(T, (H + 2 * G) * D)
            t = timed(lambda: ops.attn_decode(qd, kc2, vc2, bt, cl, H, G, D, D ** -0.5, ctx))
            add("attn_decode (split-K)", phase, t, bytes_=B * ctx * 2 * G * D * 2, like="sink_attn")
        # ---- delta rule: short convolution + recurrence + gated norm
        C = 2 * dG * dD + dH * dV
        pr = rn(T, C + dH * dV + 2 * dH)
        cw4, tail4 = rn(C, 4), torch.zeros(B, 3, C, device=dev)
        t = timed(lambda: ops.causal_conv(pr[:, :C], cw4, tail4, cu, cl, ss, False, True, torch.float32))
        add("causal_conv (4 taps, SiLU)", phase, t, bytes_=T * C * (2 + 4))
        qkv32 = rn(T, C, dt=torch.float32)
        S = torch.zeros(B, dH, dD, dV, device=dev)
        A_log, dtb = rn(dH, dt=torch.float32), rn(dH, dt=torch.float32)
        ab = pr[:, C + dH * dV:]
        f_delta = lambda: ops.delta_recurrence(qkv32[:, :dG * dD], qkv32[:, dG * dD:2 * dG * dD], qkv32[:, 2 * dG * dD:],
                                               ab[:, :dH], ab[:, dH:], A_log, dtb, S, cu, cl, ss, dH, dG, dD, dV)
        t = timed(f_delta, iters=3, warm=1)
        add("delta_recurrence", phase, t, flops=T * dH * dD * dV * 2 * 3,
            bytes_=B * dH * dD * dV * 4 * 2 + T * (C + dH * dV) * 4)
        o32 = rn(T, dH * dV, dt=torch.float32)
        nw = rn(dV)
        t = timed(lambda: ops.gated_group_norm(o32, pr[:, C:C + dH * dV], nw, 1e-6, "silu", 1.0,
                                               out=both[:, H * D:]))
        add("gated_group_norm", phase, t, bytes_=T * dH * dV * (4 + 2 + 2))
        # ---- decay linear attention
        pl = rn(T, 2 * lH * lD + 2 * lH * lV)
        S2 = torch.zeros(B, lH, lD, lV, device=dev)
        dec = torch.full((lH,), 0.97, device=dev)
        f_dec = lambda: ops.decay_recurrence(pl[:, :lH * lD], pl[:, lH * lD:2 * lH * lD],
                                             pl[:, 2 * lH * lD:2 * lH * lD + lH * lV], dec, S2, cu, cl, ss, lH, lD, lV, True)
        t = timed(f_dec, iters=3, warm=1)
        add("decay_recurrence", phase, t, flops=T * lH * lD * lV * 2 * 2,
            bytes_=B * lH * lD * lV * 4 * 2 + T * (2 * lH * lD + 2 * lH * lV) * 2)
        # ---- feed-forward: gate | up GEMM + activation + down GEMM (Llama: GEMM with the activation in its epilogue)
        h = rn(T, W)
        gu_w, dn_w = rn(2 * F, W, std=W ** -0.5), rn(W, F, std=F ** -0.5)
        f_ff = lambda: ops.linear_f(ops.glu_act(ops.linear_f(h, gu_w, bf), F, "gelu_tanh"), dn_w, bf)
        t = timed(f_ff)
        add("feed-forward (2 GEMMs + glu_act)", phase, t, flops=T * W * F * 6, bytes_=3 * W * F * 2)
        gu_i = ops.glu_interleave(gu_w[:F], gu_w[F:]).contiguous()
        if gu_i is not None:
            t = timed(lambda: ops.linear(ops.linear(h, gu_i, None, "none", True), dn_w))
            add("gated MLP (fused epilogue)", phase, t, flops=T * W * F * 6, bytes_=3 * W * F * 2, like="feed-forward")
        # ---- the mixer's input and output GEMMs
        Np = -(-(nq + nk + nv + C + dH * dV + 2 * dH) // 8) * 8
        pw = rn(Np, W, std=W ** -0.5)
        t = timed(lambda: ops.linear_f(h, pw, bf))
        add("mixer input GEMM (all projections)", phase, t, flops=T * W * Np * 2, bytes_=W * Np * 2)
        ow = rn(W, H * D + dH * dV, std=0.02)
        t = timed(lambda: ops.linear_f(both, ow, bf))
        add("mixer output GEMM (both branches)", phase, t, flops=T * W * (H * D + dH * dV) * 2,
            bytes_=W * (H * D + dH * dV) * 2)
    print(json.dumps(dict(size=a.size, shape=s, tokens=a.tokens, seq=a.seq, batch=a.batch, ctx=a.ctx, kernels=rows)))


if __name__ == "__main__":
    main()
