"""Each mechanism of the Lamisun design alone: the framework's op (CPU definition, and on a GPU box the HIP kernel in
fp32 and bf16 storage) against the plain float64 function in lamisun_oracle.py, over pages that are scattered, state
slots that held something else before, portions cut at awkward places, and inputs built so that a fault shows (a key
whose score stands out placed far back, at page borders and just inside / just outside a chunk)."""
import numpy as np
import pytest
import torch

import lamisun_oracle as oracle
from llmss_amd import ops

gpu = pytest.mark.gpu
RUNS = [pytest.param("cpu", torch.float32, id="cpu-fp32"), pytest.param("cuda", torch.float32, marks=gpu, id="gpu-fp32"),
        pytest.param("cuda", torch.bfloat16, marks=gpu, id="gpu-bf16")]
F64 = torch.float64


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def close(got, want, dtype, what="", scale=None):
    got, want = got.detach().double().cpu(), want.double()
    s = float(want.abs().max()) if scale is None else scale
    err = float((got - want).abs().max()) / max(s, 1e-9)
    assert err < tol(dtype), f"{what}: error {err:.3g} of the largest value"


def rnd(*shape, seed=0, dtype=torch.float32):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(*shape, generator=g).to(dtype).double()  # values the storage type holds exactly


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


# ------------------------------------------------------------------------------------------- embedding and residual
@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("V,W,buckets,mp,mc", [(50, 24, 13, 5, 3), (9, 40, 1, 1, 1), (300, 17, 97, 2 ** 31 - 1, 65537)])
def test_bigram_embedding_carries_the_previous_token(device, dtype, V, W, buckets, mp, mc):
    table, big = rnd(V, W, seed=1, dtype=dtype), rnd(buckets + 1, W, seed=2, dtype=dtype)
    seqs = [np.random.default_rng(3 + s).integers(0, V, n).tolist() for s, n in enumerate((23, 1, 9))]
    prev = torch.full((4,), 7, dtype=torch.int64, device=device)  # what earlier sequences left in the slots
    slots = [2, 0, 3]
    got = [torch.zeros(len(t), W) for t in seqs]
    for step in steps_of([[5, 1, 1, 2, 14], [1], [2, 1, 6]]):
        cu, ctx, ss = meta(step, slots, device)
        ids = torch.tensor(sum((seqs[s][p0:p0 + n] for s, p0, n in step), []), device=device)
        pos = torch.tensor(sum((list(range(p0, p0 + n)) for _, p0, n in step), []), device=device)
        hist = torch.full((3, len(ids), W), 9.0, device=device)
        ops.embed_bigram(ids, pos, table.to(dtype).to(device), 0.37, big.to(dtype).to(device), mp, mc, prev, cu, ctx, ss,
                         hist)
        assert torch.equal(hist[0], hist[1]) and float(hist[2].min()) == 9.0
        r = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = hist[0][r:r + n].cpu()
            r += n
    for s, t in enumerate(seqs):
        close(got[s], oracle.embed(t, table, big, 0.37, buckets, mp, mc), torch.float32, f"sequence {s}")
    assert prev.tolist() == [seqs[1][-1], 7, seqs[0][-1], seqs[2][-1]]


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("W,n,dwa", [(40, 0, False), (48, 1, True), (100, 3, True), (37, 5, True), (64, 2, False)])
def test_output_normed_residual_and_depth_average(device, dtype, W, n, dwa):
    T, eps = 6, 1e-5
    h0 = rnd(n + 2, T, W, seed=1) * 2
    y, w = (rnd(T, W, seed=2) * 3).to(dtype).double(), (1 + 0.1 * rnd(W, seed=3)).to(dtype).double()
    wd = rnd(n + 1, seed=4).float().double() if dwa else None
    hist = h0.float().to(device).contiguous()
    out = ops.resid_norm_add(hist, n, y.to(dtype).to(device), w.to(dtype).to(device), eps,
                             wd.float().to(device) if dwa else None)
    x = h0[n].float().double() + oracle.rms_div(y, eps) * w
    close(hist[n], x, torch.float32, "the layer's result")
    for j in range(n):
        assert torch.equal(hist[j].cpu(), h0[j].float()), "earlier results are left alone"
    if dwa:
        want = sum(wd[j] * (x if j == n else h0[j].float().double()) for j in range(n + 1))
        close(hist[n + 1], want, torch.float32, "depth average")
        assert out.data_ptr() == hist[n + 1].data_ptr()
    else:
        assert out.data_ptr() == hist[n].data_ptr()
        assert torch.equal(hist[n + 1].cpu(), h0[n + 1].float())


@pytest.mark.parametrize("device,dtype", RUNS)
def test_xielu_and_the_output_gate(device, dtype):
    z = torch.cat([rnd(5, 67, seed=1, dtype=dtype) * 3, torch.tensor([[0.0, -0.0, 1e-4, -1e-4, -30.0, 30.0] + [0.5] * 61])
                   .to(dtype).double()])
    p, q = 0.3, -0.7
    got = ops.act_fn(z.to(dtype).to(device), "xielu", (oracle.softplus(p), 0.5 + oracle.softplus(q)))
    close(got, oracle.xielu(z, p, q), dtype, "xIELU")
    y, src = rnd(5, 24, seed=2, dtype=dtype), rnd(5, 40, seed=3, dtype=dtype) * 4
    yd = y.to(dtype).to(device).clone()
    ops.gate_mul(yd, src.to(dtype).to(device), 11)
    close(yd, y * torch.sigmoid(src[:, 11:35]), dtype, "gate")
    # rows of whole 16-byte pieces (the wide accesses of the bf16 kernel), more columns than one pass of a workgroup
    y, src = rnd(3, 4112, seed=4, dtype=dtype), rnd(3, 4200, seed=5, dtype=dtype) * 4
    yd = y.to(dtype).to(device).clone()
    ops.gate_mul(yd, src.to(dtype).to(device), 88)
    close(yd, y * torch.sigmoid(src[:, 88:]), dtype, "gate, wide rows")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("taps", [1, 2, 3, 5])
def test_input_convolution_reads_the_fp32_residual(device, dtype, taps):
    """x + conv(x) over the fp32 residual, weights in the storage type, portions shorter than the tail."""
    C, n = 20, 19
    x, w = rnd(n, C, seed=1), rnd(C, taps, seed=2, dtype=dtype)
    state = torch.full((2, max(taps - 1, 1), C), 5.0, device=device)[:, :taps - 1].contiguous()
    got = torch.zeros(n, C)
    for step in steps_of([[1, 1, 2, 1, 6, 8]]):
        cu, ctx, ss = meta(step, [1], device)
        (_, p0, k), = step
        got[p0:p0 + k] = ops.causal_conv(x[p0:p0 + k].float().to(device), w.to(dtype).to(device),
                                         state if taps > 1 else None, cu, ctx, ss, True, False, torch.float32).cpu()
    close(got, x.float().double() + oracle.causal_conv(x.float().double(), w), torch.float32, "x + conv(x)")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("taps", [1, 2, 4, 9, 12])
@pytest.mark.parametrize("C", [300, 21])
def test_input_convolution_over_long_portions(device, dtype, taps, C):
    """Steps of several hundred rows (on a GPU the kernel that walks strips of rows): sequences of unequal length
    side by side, sequence ends inside a strip and at its first row, an empty portion's neighbour, portions that
    continue from the tail, and widths that are no multiple of the workgroup or of a 16-byte read."""
    lens = [333, 17, 290, 64]
    cuts = [[16, 317], [16, 1], [290], [48, 16]]  # 370 rows of four sequences, then 334 rows of three
    xs = [rnd(n, C, seed=10 + i) for i, n in enumerate(lens)]
    w = rnd(C, taps, seed=2, dtype=dtype)
    state = torch.full((4, max(taps - 1, 1), C), -3.0, device=device)[:, :taps - 1].contiguous()
    got = [torch.zeros(n, C) for n in lens]
    for step in steps_of(cuts):
        cu, ctx, ss = meta(step, [2, 0, 3, 1], device)
        x = torch.cat([xs[s][p0:p0 + k] for s, p0, k in step]).float().to(device)
        y = ops.causal_conv(x, w.to(dtype).to(device), state if taps > 1 else None, cu, ctx, ss, True, False,
                            torch.float32).cpu()
        at = 0
        for s, p0, k in step:
            got[s][p0:p0 + k] = y[at:at + k]
            at += k
    for s, n in enumerate(lens):
        close(got[s], xs[s].float().double() + oracle.causal_conv(xs[s].float().double(), w), torch.float32,
              f"x + conv(x), sequence {s}")


# ------------------------------------------------------------------------------------------------- latent attention
@pytest.mark.parametrize("base,rot", [(10000.0, 8), (250000.0, 16), (20.0, 2)])
@pytest.mark.parametrize("device", ["cpu", pytest.param("cuda", marks=gpu)])
def test_angles_of_far_positions(device, base, rot):
    pos = torch.tensor([0, 1, 2, 17, 1000, 4099, 65537, 999983], device=device)
    f = torch.tensor([base ** (-2.0 * i / rot) for i in range(rot // 2)], dtype=F64)
    cs = ops.rope_angles(pos, f.float().to(device)).cpu().double()
    ang = pos.cpu().float()[:, None].double() * f.float().double()[None]  # the fp32 product is the angle
    ang32 = (pos.cpu().float()[:, None] * f.float()[None]).double()
    assert float((cs[..., 0] - torch.cos(ang32)).abs().max()) < 2e-7
    assert float((cs[..., 1] - torch.sin(ang32)).abs().max()) < 2e-7
    assert float((cs[..., 0] - torch.cos(ang)).abs().max()) < 0.05  # and that product is near the exact one


def latent_case(device, dtype, H, d, r, dv, R, lens, cuts, scale, base=1000.0, bs=16, boost=None, seed=0):
    """The latent mixer between its projections: norm + rotation + cache write, absorbed queries, attention over the
    pages, value expansion. ``boost`` = (sequence, key position, factor): the last two queries are aligned with that
    key's latent, which is made long, so that nearly all their weight sits there."""
    eps = 1e-5
    pg = Pages(lens, bs, device, seed)
    cache = torch.zeros(pg.blocks, bs, R + r, dtype=dtype, device=device)
    uk, uv = rnd(H * d, R, seed=seed + 50, dtype=dtype) * R ** -0.5, rnd(H * dv, R, seed=seed + 51, dtype=dtype) * R ** -0.5
    nw = (1 + 0.1 * rnd(R, seed=seed + 52)).to(dtype).double()
    f = torch.tensor([base ** (-2.0 * i / r) for i in range(r // 2)], dtype=F64).float().to(device) if r else None
    data = []
    for i, n in enumerate(lens):
        q, down = rnd(n, H * (d + r), seed=seed + 2 * i + 1, dtype=dtype), rnd(n, R + r, seed=seed + 2 * i + 2, dtype=dtype)
        if boost and boost[0] == i:
            c = oracle.rms_div(down[boost[1], :R], eps) * nw
            for row in (-1, -2):  # the absorbed query becomes that latent's projection onto the rows of W_uk
                qh = q[row].view(H, d + r)
                for a, m in enumerate(uk.view(H, d, R)):
                    qh[a, :d] = (boost[2] * torch.linalg.solve(m @ m.T, m @ c)).to(dtype).double()
                qh[:, d:] = 0
        data.append((q, down))
    uk_t = uk.view(H, d, R).transpose(1, 2).contiguous().to(dtype).to(device)
    got = [torch.zeros(n, H * dv) for n in lens]
    for step in steps_of(cuts):
        step = sorted(step, key=lambda e: not (e[2] == 1 and e[1] > 0))
        seqs = [s for s, _, _ in step]
        cu, ctx, _ = meta(step, [0] * len(lens), device)
        src = torch.cat([torch.cat([data[s][0][p0:p0 + n], data[s][1][p0:p0 + n]], 1) for s, p0, n in step])
        src = src.to(dtype).to(device)
        pos = torch.tensor(sum((list(range(p0, p0 + n)) for _, p0, n in step), []), device=device)
        slots = torch.tensor(sum((pg.slots(s, p0, n) for s, p0, n in step), []), device=device)
        qa = ops.head_absorb(src, uk_t, ops.latent_qa_dtype(cache), extra=r)
        cs = ops.rope_angles(pos, f) if r else None
        ops.latent_norm_cache(src, H * (d + r), R, nw.to(dtype).to(device), eps, cache, slots, r, cs,
                              qa if r else None, 0, d)
        single = all(n == 1 for _, _, n in step)
        o = ops.latent_attn(qa, cache, pg.bt(seqs), cu, ctx, 0, scale, max_qlen=max(n for _, _, n in step),
                            max_ctx=max(lens) if single else 0)
        y = ops.head_expand(o, uv.to(dtype).to(device), torch.float32).cpu()
        k = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = y[k:k + n]
            k += n
    for s, n in enumerate(lens):
        want = oracle.latent_heads(data[s][0], data[s][1], nw, uk, uv, H, d, r, dv, R, base, scale, eps)
        close(got[s], want, dtype, f"sequence {s}", scale=float(want.abs().max()))
    return got, data, (uk, uv, nw)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,d,r,dv,R", [(3, 8, 4, 12, 20), (1, 16, 2, 8, 8), (4, 32, 16, 32, 48), (2, 64, 32, 40, 96),
                                        (2, 24, 64, 16, 192), (5, 6, 6, 7, 10)])
def test_latent_attention_portions_decoding_and_batches(device, dtype, H, d, r, dv, R):
    # cached rows of 64 / 128 / 256 numbers: in bf16 on a GPU the matrix-core kernel runs
    latent_case(device, dtype, H, d, r, dv, R, [70, 1, 33], [[16, 1, 15, 2, 1, 1, 30, 3, 1], [1], [2, 31]], 0.3)
    latent_case(device, dtype, H, d, r, dv, R, [150, 90], [[65, 64, 1, 20], [3, 87]], 0.2, base=50.0, seed=7)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("R,r", [(20, 4), (96, 32)])
@pytest.mark.parametrize("far", [0, 15, 16, 17, 63, 64, 200])
def test_a_far_latent_row_among_hundreds(device, dtype, far, R, r):
    H, d, dv, n = 2, 32, 8, 300
    got, data, (uk, uv, nw) = latent_case(device, dtype, H, d, r, dv, R, [n], [[n - 1, 1]], 0.3, boost=(0, far, 9.0),
                                          seed=100 + far)
    c = oracle.rms_div(data[0][1][:, :R], 1e-5) * nw
    s = ((data[0][0][-1].view(H, d + r)[0, :d] @ uk.view(H, d, R)[0]) @ c.T) * 0.3
    w = torch.softmax(s, -1)
    assert int(s.argmax()) == far and float(w[far]) > 0.9  # nearly all of the row's weight sits on that key
    v_far = (uv.view(H, dv, R)[0] @ c[far])
    for row in (-1, -2):  # the decoded token and the prompt's last row
        assert float((got[0][row].view(H, dv)[0].double() - v_far).abs().max()) < 0.2 * float(v_far.abs().max()) + 0.05


# ------------------------------------------------------------------------------------------ differential attention
def two_map_case(device, dtype, H, G, d, dv, lens, cuts, scale, lam, chunk, bs=16, boost=None, seed=0, norm=True):
    """Query / key norm + cache write, the two maps over the pages (no sink, chunked mask, two key heads per value
    head), their combination. ``boost`` = (sequence, key position, factor, query rows): map 0 of those queries points
    along that key."""
    eps, mult = 1e-5, 0.65
    pg = Pages(lens, bs, device, seed)
    kc = torch.zeros(pg.blocks, bs, G * 2 * d, dtype=dtype, device=device)
    vc = torch.zeros(pg.blocks, bs, G * dv, dtype=dtype, device=device)
    qw, kw = (1 + 0.2 * rnd(d, seed=seed + 60)).to(dtype).double(), (1 + 0.2 * rnd(d, seed=seed + 61)).to(dtype).double()
    nq, nk, nv = H * 2 * d, G * 2 * d, G * dv
    data = []
    for i, n in enumerate(lens):
        q, k, v = rnd(n, H, 2, d, seed=seed + 3 * i + 1, dtype=dtype), rnd(n, G, 2, d, seed=seed + 3 * i + 2, dtype=dtype), \
            rnd(n, G, dv, seed=seed + 3 * i + 3, dtype=dtype)
        if boost and boost[0] == i:
            for row in boost[3]:
                q[row, :, 0] = (boost[2] * k[boost[1], :, 0]).repeat_interleave(H // G, 0)
            k[boost[1], :, 0] *= 2  # and the key is made long
        data.append((q, k, v))
    got = [torch.zeros(n, H * dv) for n in lens]
    for step in steps_of(cuts):
        step = sorted(step, key=lambda e: not (e[2] == 1 and e[1] > 0))  # single rows after a prefix come first
        nd = sum(1 for _, p0, n in step if n == 1 and p0 > 0)
        seqs = [s for s, _, _ in step]
        cu, ctx, _ = meta(step, [0] * len(lens), device)
        proj = torch.cat([torch.cat([torch.zeros(n, 3, dtype=F64)] + [x[p0:p0 + n].reshape(n, -1) for x in data[s]], 1)
                          for s, p0, n in step]).to(dtype).to(device)
        slots = torch.tensor(sum((pg.slots(s, p0, n) for s, p0, n in step), []), device=device)
        q = ops.qk_norm_cache(proj, 3, 3 + nq, 3 + nq + nk, qw.to(dtype).to(device) if norm else None,
                              kw.to(dtype).to(device) if norm else None, eps, kc, vc, slots, H, G, 2, d, dv)
        single = nd == len(step)
        O = ops.sink_attn(q, kc, vc, pg.bt(seqs), cu, ctx, 2 * H, 2 * G, d, dv, scale, 0.0, False,
                          max_qlen=1 if single else max(n for _, _, n in step), num_decode=0 if single else nd,
                          sink=False, chunk=chunk, vshare=2, precise=True)
        y = ops.diff_combine(O, lam, eps, mult, H, G, dv, torch.float32).cpu()
        r = 0
        for s, p0, n in step:
            got[s][p0:p0 + n] = y[r:r + n]
            r += n
    for s, n in enumerate(lens):
        q, k, v = data[s]
        if norm:
            q, k = oracle.rms_div(q, eps) * qw, oracle.rms_div(k, eps) * kw
        want = oracle.two_map_heads(q, k, v, scale, lam, mult, chunk, eps)
        close(got[s], want, dtype, f"sequence {s}", scale=float(want.abs().max()))
    return got, data


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,d,dv,chunk", [(4, 2, 8, 12, 10), (4, 4, 8, 20, 7), (3, 1, 24, 40, 0), (1, 1, 8, 8, 1),
                                            (8, 2, 64, 72, 48), (16, 2, 32, 8, 33), (4, 2, 128, 64, 64),
                                            (4, 1, 128, 40, 100), (6, 2, 64, 160, 16), (2, 2, 32, 128, 0),
                                            (6, 3, 6, 5, 5)])
def test_two_map_attention_portions_decoding_and_batches(device, dtype, H, G, d, dv, chunk):
    # key sizes 32, 64, 128 with value sizes in eights: in bf16 on a GPU the portions run on the matrix cores
    two_map_case(device, dtype, H, G, d, dv, [70, 1, 33], [[16, 1, 15, 2, 1, 1, 30, 3, 1], [1], [2, 31]], d ** -0.5,
                 0.55, chunk)
    two_map_case(device, dtype, H, G, d, dv, [150, 90], [[65, 64, 1, 20], [3, 87]], d ** -0.5, -0.3, chunk, seed=7,
                 norm=False)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("H,G,d,dv,chunk", [(8, 2, 64, 128, 100), (4, 4, 32, 64, 0), (6, 2, 128, 48, 128),
                                            (3, 1, 64, 40, 77)])
def test_two_map_attention_over_long_portions(device, dtype, H, G, d, dv, chunk):
    """Portions of hundreds of rows beside a shorter one: many row blocks per sequence (on the matrix cores a wave
    holds two groups of rows there), key tiles that every row of a group sees whole and tiles cut by the diagonal
    or by a chunk's first position, a portion that continues far into its sequence."""
    two_map_case(device, dtype, H, G, d, dv, [333, 140, 9], [[200, 133], [140], [9]], d ** -0.5, 0.45, chunk, seed=11)


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("d", [16, 64])
@pytest.mark.parametrize("chunk,key,row", [(48, 96, 143), (48, 95, 143), (48, 144, 144), (48, 143, 144), (64, 128, 191),
                                           (64, 127, 191), (10, 190, 199), (10, 189, 199), (0, 0, 199), (0, 17, 199)])
def test_a_key_just_inside_and_just_outside_a_chunk(device, dtype, d, chunk, key, row):
    """One key's score is made to stand out for the query at ``row``: inside the row's chunk it takes nearly all
    the weight of map 0, one position before the chunk's first it must leave no trace. The row is once the last of
    a prompt portion and once a single decoded token."""
    H, G, dv, n = 2, 1, 8, 203
    inside = key >= (row // chunk * chunk if chunk else 0)
    for cuts in ([row + 1, n - row - 1], [row, 1, n - row - 1], [key + 1, row - key - 1, 1, 1, n - row - 2] if key + 1 < row
                 else [row, 1, n - row - 1]):
        cuts = [c for c in cuts if c > 0]
        got, data = two_map_case(device, dtype, H, G, d, dv, [n], [cuts], 0.5, 0.0, chunk, boost=(0, key, 3.0, [row]),
                                 seed=200 + key, norm=False)
        q, k, v = data[0]
        lo = row // chunk * chunk if chunk else 0
        s = (q[row, 0, 0] @ k[lo:row + 1, 0, 0].T) * 0.5
        w = torch.softmax(s, -1)
        o = got[0][row].view(H, dv)[0].double()
        if inside:  # lam = 0: the head is map 0's output, normed; nearly all of it is that key's value row
            assert int(s.argmax()) == key - lo and float(w[key - lo]) > 0.9
            want = oracle.rms_div(v[key, 0], 1e-5) * 0.65
            assert float((o - want).abs().max()) < 0.25
        else:
            assert key < lo


@pytest.mark.parametrize("device,dtype", RUNS)
def test_second_map_is_subtracted_with_the_layers_weight(device, dtype):
    """Both maps see the same values; with lam = 1 and equal maps the difference vanishes before the norm, so the
    maps are made unequal and lam is varied: the result follows the oracle for lam of either sign and size."""
    for lam in (0.0, 1.0, -2.5, 0.37):
        two_map_case(device, dtype, 4, 2, 16, 12, [40], [[13, 1, 26]], 0.3, lam, 9, seed=int(10 * abs(lam)))
