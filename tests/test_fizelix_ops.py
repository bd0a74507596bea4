"""Each mechanism of the Fizelix design alone: the framework's op (CPU definition, and on a GPU box the HIP kernel in
fp32 and bf16 storage) against the plain float64 function in fizelix_oracle.py, over pages that are scattered, state
slots that held something else before, portions cut at awkward places, and inputs built so that a fault shows (a key
whose score stands out placed far back in a pooled block, at page borders, just inside / just outside the window and
in a block that is just pooled / not yet pooled)."""
import numpy as np
import pytest
import torch

import fizelix_oracle as oracle
from llmss_amd import ops

gpu = pytest.mark.gpu
RUNS = [pytest.param("cpu", torch.float32, id="cpu-fp32"), pytest.param("cuda", torch.float32, marks=gpu, id="gpu-fp32"),
        pytest.param("cuda", torch.bfloat16, marks=gpu, id="gpu-bf16")]
F64 = torch.float64


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def close(got, want, dtype, what="", scale=None, slack=1.0):
    got, want = got.detach().double().cpu(), want.double()
    s = float(want.abs().max()) if scale is None else scale
    err = float((got - want).abs().max()) / max(s, 1e-9)
    assert err < tol(dtype) * slack, f"{what}: error {err:.3g} of the largest value"


def rnd(*shape, seed=0, dtype=torch.float32, mul=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * mul).to(dtype).double()  # values the storage type holds exactly


def i32(x, device):
    return torch.tensor(x, dtype=torch.int32, device=device)


def steps_of(cuts_per_seq):
    """[(seq, first position, rows)] step lists: step k feeds portion k of every sequence that still has one."""
    at = [0] * len(cuts_per_seq)
    out = []
    for k in range(max(len(c) for c in cuts_per_seq)):
        step = []
        for s, cuts in enumerate(cuts_per_seq):
            if k < len(cuts):
                step.append((s, at[s], cuts[k]))
                at[s] += cuts[k]
        out.append(step)
    return out


def meta(step, slots, device):
    cu = np.cumsum([0] + [n for _, _, n in step])
    return (i32(cu.tolist(), device), i32([p0 + n for _, p0, n in step], device), i32([slots[s] for s, _, _ in step], device))


class Pages:
    """Block tables over a pool whose pages are handed out in a scrambled order."""

    def __init__(self, lens, bs, device, seed):
        self.bs = bs
        need = [-(-n // bs) for n in lens]
        order = np.random.default_rng(seed).permutation(sum(need) + 3).tolist()
        self.tables, at = [], 0
        for n in need:
            self.tables.append(order[at:at + n])
            at += n
        self.blocks = sum(need) + 3
        self.device = device

    def slots(self, s, p0, n):
        return [self.tables[s][p // self.bs] * self.bs + p % self.bs for p in range(p0, p0 + n)]

    def bt(self, seqs):
        w = max(len(t) for t in self.tables)
        return i32([self.tables[s] + [0] * (w - len(self.tables[s])) for s in seqs], self.device)


# ------------------------------------------------------------------------------------------- the block's closing ops
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("W", [48, 50, 264])
def test_sandwich_add_norm(device, dtype, W):
    T, eps = 7, 1e-5
    x, y, h = rnd(T, W, seed=1, mul=2.0), rnd(T, W, seed=2, dtype=dtype), rnd(T, W, seed=3, dtype=dtype)
    rg, rgb = rnd(W, W, seed=4, dtype=dtype, mul=W ** -0.5), rnd(W, seed=5, mul=0.3)
    nb, ls, nn, add = 1 + 0.1 * rnd(W, seed=6), 0.5 + 0.1 * rnd(W, seed=7), 1 + 0.1 * rnd(W, seed=8), rnd(T, W, seed=9)
    r = (h @ rg.T).to(dtype).double()  # the gate logits as the projection leaves them
    gated = oracle.rms(y * torch.sigmoid(r + rgb), eps) * nb * ls
    dev = lambda t, dt=torch.float32: t.to(device=device, dtype=dt).contiguous()
    # the logits are columns of a wider projection: rows are strided
    wide = torch.zeros(T, W + 8, dtype=dtype, device=device)
    wide[:, 8:] = dev(r, dtype)
    for use_gate, use_add, use_next in ((True, False, True), (False, True, True), (True, True, False)):
        xs = dev(x)
        want = x + (gated if use_gate else oracle.rms(y, eps) * nb * ls) + (add if use_add else 0)
        got = ops.sandwich_add_norm(xs, dev(y, dtype), wide[:, 8:] if use_gate else None, dev(rgb) if use_gate else None,
                                    dev(nb * ls), eps, dev(add) if use_add else None, dev(nn) if use_next else None, dtype)
        close(xs, want, torch.float32, "residual", slack=1.0 if dtype == torch.float32 else 50.0)
        if use_next:
            close(got, oracle.rms(want, eps) * nn, dtype, "next input")
        else:
            assert got is None
    xs = dev(x)  # no sublayer at all: the embedding comes back in, then the norm
    got = ops.sandwich_add_norm(xs, None, None, None, None, eps, dev(add), dev(nn), dtype)
    close(xs, x + add, torch.float32, "re-added embedding")
    close(got, oracle.rms(x + add, eps) * nn, dtype, "norm after it")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("W,d,part", [(48, 6, 2), (50, 1, 0), (264, 19, 1)])
def test_token_side_add(device, dtype, W, d, part):
    T, V, eps = 9, 31, 1e-5
    x = rnd(T, W, seed=1, mul=2.0)
    table, gate, proj = rnd(V, 3 * d, seed=2, dtype=dtype), rnd(d, W, seed=3, dtype=dtype, mul=W ** -0.5), rnd(W, d, seed=4, dtype=dtype)
    norm, nn, add = 1 + 0.1 * rnd(W, seed=5), 1 + 0.1 * rnd(W, seed=6), rnd(T, W, seed=7)
    ids = torch.tensor([0, 30, 5, 5, 17, 2, 29, 1, 8])
    want = x + oracle.token_side(x, table[ids][:, part * d:(part + 1) * d], gate, proj, norm, eps)
    dev = lambda t, dt=torch.float32: t.to(device=device, dtype=dt).contiguous()
    xs = dev(x)
    got = ops.token_side_add(xs, ids.to(device), dev(table, dtype), part * d, dev(gate, dtype), dev(proj, dtype), dev(norm),
                             eps, None, dev(nn), dtype)
    close(xs, want, torch.float32, "residual", slack=1.0 if dtype == torch.float32 else 5.0)
    close(got, oracle.rms(want, eps) * nn, dtype, "next input")
    xs = dev(x)
    assert ops.token_side_add(xs, ids.to(device), dev(table, dtype), part * d, dev(gate, dtype), dev(proj, dtype), dev(norm),
                              eps, dev(add), None, dtype) is None
    close(xs, want + add, torch.float32, "residual with the embedding re-added", slack=1.0 if dtype == torch.float32 else 5.0)


# -------------------------------------------------------------------------- windowed sigmoid attention, pooled blocks
def run_attention(device, dtype, lens, cuts, H, G, dim, vdim, window, pool, rot, bs=16, seed=0, q=None, k=None, v=None,
                  scale=0.3, pb=None, max_ctx=0):
    """Feeds q / k / v rows of several sequences through rope_pairs_cache, pool_update and pool_window_attn step by
    step (portions as ``cuts`` says, all sequences of a step in one batch) and returns per sequence (got, want)."""
    S = len(lens)
    base = 1000.0
    if q is None:
        q = [rnd(n, H * dim, seed=seed + 10 * s + 1, dtype=dtype) for s, n in enumerate(lens)]
        k = [rnd(n, G * dim, seed=seed + 10 * s + 2, dtype=dtype) for s, n in enumerate(lens)]
        v = [rnd(n, G * vdim, seed=seed + 10 * s + 3, dtype=dtype) for s, n in enumerate(lens)]
    pb = pb if pb is not None else rnd(H, seed=seed + 7, mul=0.5)
    pages = Pages(lens, bs, device, seed)
    kc = torch.full((pages.blocks, bs, G * dim), 7.0, dtype=dtype, device=device)  # stale values everywhere
    vc = torch.full((pages.blocks, bs, G * vdim), -3.0, dtype=dtype, device=device)
    per = -(-bs // pool) if pool else 0
    kp = torch.full((pages.blocks, per, G * dim), 5.0, dtype=dtype, device=device) if pool else None
    vp = torch.full((pages.blocks, per, G * vdim), 5.0, dtype=dtype, device=device) if pool else None
    freqs = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=torch.float32, device=device) if rot else None
    got = [torch.zeros(n, H * vdim, dtype=F64) for n in lens]
    for step in steps_of(cuts):
        rows = torch.cat([torch.cat([q[s][p0:p0 + n], k[s][p0:p0 + n], v[s][p0:p0 + n]], 1) for s, p0, n in step])
        pos = torch.cat([torch.arange(p0, p0 + n) for _, p0, n in step]).to(device)
        slots = torch.tensor(sum((pages.slots(s, p0, n) for s, p0, n in step), []), dtype=torch.int64, device=device)
        cu, ctx, _ = meta(step, list(range(S)), device)
        cs = ops.rope_angles(pos, freqs) if rot else None
        proj = rows.to(device=device, dtype=dtype)
        qq = ops.rope_pairs_cache(proj, 0, H * dim, (H + G) * dim, cs, kc, vc, slots, H, G, dim, vdim)
        bt = pages.bt([s for s, _, _ in step])
        mq = max(n for _, _, n in step)
        if pool:
            ops.pool_update(kc, vc, kp, vp, bt, cu, ctx, pool, max_qlen=mq)
        out = ops.pool_window_attn(qq, kc, vc, kp, vp, bt, cu, ctx, pb.float().to(device), H, G, dim, vdim, scale,
                                   window, pool, torch.float32, max_qlen=mq, max_ctx=max_ctx)
        at = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = out[at:at + n].double().cpu()
            at += n
    res = []
    for s, n in enumerate(lens):
        p = torch.arange(n)
        qr = oracle.rotate_pairs(q[s].view(n, H, dim), p, rot, base) if rot else q[s].view(n, H, dim)
        kr = oracle.rotate_pairs(k[s].view(n, G, dim), p, rot, base) if rot else k[s].view(n, G, dim)
        kr = kr.to(dtype).double()  # keys as the cache holds them
        want = oracle.window_pool_attention(qr, kr, v[s].view(n, G, vdim), pb, scale, window, pool)
        res.append((got[s], want.reshape(n, H * vdim)))
    return res


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,dim,vdim,window,pool,rot", [
    (4, 2, 8, 12, 7, 3, 4),      # the pool does not divide the page, grouped heads, partial rotation
    (3, 3, 6, 5, 5, 1, 6),       # blocks of one position, every head its own keys, whole head rotated
    (2, 1, 16, 8, 4, 16, 0),     # a block as long as a page, longer than the window, no rotation
    (8, 1, 4, 70, 9, 5, 2),      # eight heads on one key head, a value row wider than a wave
    (2, 2, 10, 6, 40, 8, 0),     # a window longer than most of the prompt
    (2, 1, 8, 8, 0, 0, 4),       # no window, no pool: every earlier position
    (2, 2, 8, 8, 6, 0, 0),       # a window without pooled blocks
    (4, 2, 32, 64, 7, 3, 8),     # sizes the matrix-core kernel takes (bf16 pages): two slot groups per wave
    (8, 2, 64, 24, 12, 5, 64),   # four heads to a key head, a value size that is no multiple of 16
    (4, 1, 128, 128, 9, 16, 32),  # the widest key, one slot group
    (2, 2, 64, 136, 20, 1, 0),   # a value row in the widest tile, blocks of one position
    (3, 1, 32, 8, 0, 0, 16),     # three heads to a key head, every earlier position
    (2, 1, 8, 8, 5, 20, 0),      # a block longer than a page (vector kernel)
    (2, 1, 64, 32, 5, 20, 0),    # the same on the matrix cores
])
def test_attention_portions_batches(device, dtype, H, G, dim, vdim, window, pool, rot):
    lens = [45, 23, 1, 38]
    cuts = [[45], [2, 2, 3, 16], [1], [30, 1, 1, 1, 1, 1, 1, 1, 1]]  # whole, small portions, one token, prompt + decoding
    for max_ctx in (0, 4096):  # with a bound on the context a step of single rows splits their keys over workgroups
        for got, want in run_attention(device, dtype, lens, cuts, H, G, dim, vdim, window, pool, rot, max_ctx=max_ctx,
                                       scale=0.3 * (8.0 / dim) ** 0.5):
            close(got, want, dtype, "attention rows", slack=1.0 if dtype == torch.float32 else 2.0)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("dim,vdim", [(8, 4), (32, 8)])
def test_attention_standout_key(device, dtype, decode, dim, vdim):
    """One key is made to match the last row's query far better than any other; its value is unlike every other. Where
    it sits decides what the last row must return: inside the window its own value, in a pooled block a P-th of it
    (through the block's mean key), in a block not yet pooled and already outside the window nothing at all."""
    H, G, window, pool, n = 2, 1, 10, 4, 90
    for place in (0, 3, 4, 15, 16, 17, 63, 64, 71, 72, 75, 76, 79, 80, 81, 89):
        q, k, v = rnd(n, H * dim, seed=1, mul=0.1), rnd(n, G * dim, seed=2, mul=0.1), rnd(n, G * vdim, seed=3, mul=0.1)
        k[place] = 0.0
        k[place, :8] = 4.0
        q[n - 1] = 0.0
        q[n - 1, :8] = 4.0
        q[n - 1, dim:dim + 8] = 4.0
        v[place] = 0.0
        v[place, :4] = torch.tensor([100.0, -50.0, 25.0, 10.0], dtype=F64)
        cuts = [[n - 6] + [1] * 6] if decode else [[n - 30, 17, 11, 2]]
        (got, want), = run_attention(device, dtype, [n], cuts, H, G, dim, vdim, window, pool, 0, q=[q.to(dtype).double()],
                                     k=[k.to(dtype).double()], v=[v.to(dtype).double()], scale=0.5,
                                     pb=torch.tensor([-6.0, -6.0], dtype=F64), max_ctx=128 if decode else 0)
        last = want[n - 1].view(H, vdim)[0, 0]
        i = n - 1
        if i - place < window:
            assert last > 90.0  # seen as a token
        elif (place // pool) * pool + pool - 1 <= i - window:
            assert 5.0 < last < 30.0  # seen through its block's mean
        else:
            assert abs(last) < 1.0  # left the window, its block not yet whole behind it
        close(got, want, dtype, f"key at {place}", slack=1.0 if dtype == torch.float32 else 2.0)


# ------------------------------------------------------------------------------------------------ state-space mixer
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("taps,C", [(3, 20), (1, 7), (4, 130)])
def test_conv_bias_silu(device, dtype, taps, C):
    lens, cuts = [30, 9, 14], [[30], [1, 2, 6], [10, 1, 1, 1, 1]]
    xs = [rnd(n, C, seed=s + 1, dtype=dtype) for s, n in enumerate(lens)]
    w, b = rnd(C, taps, seed=8, dtype=dtype, mul=taps ** -0.5), rnd(C, seed=9, dtype=dtype, mul=0.3)
    state = torch.full((5, max(taps - 1, 0), C), 9.0, device=device)  # slots that held something else
    slots = [3, 0, 4]
    got = [torch.zeros(n, C, dtype=F64) for n in lens]
    for step in steps_of(cuts):
        cu, ctx, ss = meta(step, slots, device)
        rows = torch.cat([xs[s][p0:p0 + n] for s, p0, n in step]).to(device=device, dtype=dtype)
        out = ops.causal_conv(rows, w.to(device=device, dtype=dtype), state, cu, ctx, ss, False, True, torch.float32,
                              bias=b.to(device=device, dtype=dtype))
        at = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = out[at:at + n].double().cpu()
            at += n
    for s in range(len(lens)):
        close(got[s], oracle.silu(oracle.causal_conv(xs[s], w, b)), torch.float32, f"sequence {s}")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("heads,groups,N,vdim", [(4, 2, 8, 12), (3, 1, 12, 16), (2, 2, 40, 5), (8, 1, 32, 70)])
def test_ssd_recurrence(device, dtype, heads, groups, N, vdim):
    lens, cuts = [40, 9, 17], [[40], [1, 2, 6], [10, 1, 1, 1, 1, 1, 1, 1]]
    x = [rnd(n, heads * vdim, seed=s + 1, dtype=dtype) for s, n in enumerate(lens)]
    Bm = [rnd(n, groups * N, seed=s + 11, dtype=dtype, mul=N ** -0.5) for s, n in enumerate(lens)]
    Cm = [rnd(n, groups * N, seed=s + 21, dtype=dtype) for s, n in enumerate(lens)]
    dt = [rnd(n, heads, seed=s + 31, dtype=dtype, mul=2.0) for s, n in enumerate(lens)]
    dt[0][5] = 30.0  # a step so large that the old state is forgotten; softplus is the identity there
    A_log, dtb, D = rnd(heads, seed=41, mul=0.5) - 0.5, rnd(heads, seed=42, mul=0.5), 1 + 0.2 * rnd(heads, seed=43)
    state = torch.full((5, heads, N, vdim), 9.0, device=device)
    slots = [3, 0, 4]
    got = [torch.zeros(n, heads * vdim, dtype=F64) for n in lens]
    f = lambda t: t.float().to(device)
    for step in steps_of(cuts):
        cu, ctx, ss = meta(step, slots, device)
        cat = lambda a: torch.cat([a[s][p0:p0 + n] for s, p0, n in step]).to(device=device, dtype=dtype)
        wide = torch.cat([cat(x), cat(Bm), cat(Cm), cat(dt)], 1)  # columns of one projection, as the mixer has them
        a, b = heads * vdim, heads * vdim + groups * N
        out = ops.ssd_recurrence(wide[:, :a], wide[:, a:b], wide[:, b:b + groups * N], wide[:, b + groups * N:], f(A_log),
                                 f(dtb), f(D), state, cu, ctx, ss, heads, groups, N, vdim)
        at = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = out[at:at + n].double().cpu()
            at += n
    for s, n in enumerate(lens):
        want = oracle.ssd_scan(x[s].view(n, heads, vdim), Bm[s].view(n, groups, N), Cm[s].view(n, groups, N),
                               oracle.softplus(dt[s] + dtb.float().double()), A_log.float().double(), D.float().double(),
                               heads, groups)
        close(got[s], want.reshape(n, -1), torch.float32, f"sequence {s}", slack=5.0)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("N,groups", [(48, 1), (48, 2), (51, 3), (320, 4)])
def test_gate_before_group_norm(device, dtype, N, groups):
    T, eps = 6, 1e-5
    y, z, w = rnd(T, N, seed=1), rnd(T, N, seed=2, dtype=dtype), 1 + 0.1 * rnd(N, seed=3, dtype=dtype)
    want = oracle.rms((y * oracle.silu(z)).view(T, groups, N // groups), eps).reshape(T, N) * w
    dev = lambda t, dt: t.to(device=device, dtype=dt).contiguous()
    got = ops.gated_group_norm(dev(y, torch.float32), dev(z, dtype), dev(w, dtype), eps, "silu", 1.0, out_dtype=dtype,
                               groups=groups, gate_first=True)
    close(got, want, dtype, "gated, then normed")
    # and the order matters: the norm-first form of the other designs gives something else
    other = ops.gated_group_norm(dev(y, torch.float32), dev(z, dtype), dev(w, dtype), eps, "silu", 1.0, out_dtype=dtype,
                                 groups=groups)
    assert float((other.double().cpu() - want).abs().max()) > 0.05


# ------------------------------------------------------------------------------------------------ mixture of experts
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("E,top,W,F,Fs", [(5, 2, 48, 20, 12), (12, 1, 32, 24, 0), (3, 3, 40, 9, 7)])
def test_moe_weight_on_input(device, dtype, E, top, W, F, Fs):
    T = 70
    h = rnd(T, W, seed=1, dtype=dtype)
    w = {"router": rnd(E, W, seed=2, dtype=dtype, mul=2.0 * W ** -0.5)}
    w["router"][E - 1] = (-w["router"][0] * 3 - 1.0).to(dtype).double()  # an expert nobody (or hardly anybody) chooses
    for e in range(E):
        w[f"e{e}.gate"], w[f"e{e}.up"] = rnd(F, W, seed=10 + e, dtype=dtype, mul=W ** -0.5), rnd(F, W, seed=30 + e, dtype=dtype, mul=W ** -0.5)
        w[f"e{e}.down"] = rnd(W, F, seed=50 + e, dtype=dtype, mul=F ** -0.5)
    if Fs:
        w["shared.gate"], w["shared.up"] = rnd(Fs, W, seed=70, dtype=dtype, mul=W ** -0.5), rnd(Fs, W, seed=71, dtype=dtype, mul=W ** -0.5)
        w["shared.down"] = rnd(W, Fs, seed=72, dtype=dtype, mul=Fs ** -0.5)
    f = {"router": {"top": top}, "shared": {"ff": Fs} if Fs else None}
    want = oracle.moe(w, "", f, h)
    dev = lambda t: t.to(device=device, dtype=dtype).contiguous()
    hd = dev(h)
    idx, wts = ops.moe_router(hd, dev(w["router"]), None, top, False)
    s = torch.sigmoid(h @ w["router"].T)
    close(wts.sort(-1).values, s.topk(top, -1).values.sort(-1).values, torch.float32, "unnormalised scores", slack=5.0)
    sh = None
    if Fs:
        gu = ops.linear_f(hd, dev(torch.cat([w["shared.gate"], w["shared.up"]])), dtype)
        sh = ops.linear_f(ops.glu_act(gu, Fs, "silu"), dev(w["shared.down"]), dtype)
    stack = lambda n: dev(torch.stack([w[f"e{e}.{n}"] for e in range(E)]))
    for combine in (True, False):
        y = ops.moe_experts(hd, idx, wts, stack("gate"), stack("up"), stack("down"), 0.0, 1.702, shared=sh,
                            combine=combine, act="silu", weight_input=True)
        if not isinstance(y, torch.Tensor):  # the GPU's uncombined form: summed inside the block's closing op
            x = torch.zeros(T, W, device=device)
            ops.sandwich_add_norm(x, y, None, None, torch.ones(W, device=device), 0.0, None, None, dtype)
            y, ref = x, oracle.rms(want, 0.0)
        else:
            ref = want
        close(y, ref, dtype, f"experts, combine={combine}", slack=1.0 if dtype == torch.float32 else 2.0)
