"""Lamisun through the framework (config reader, checkpoint loader, engine, scheduler, paged cache, state slots,
kernels) against the plain float64 definition in lamisun_oracle.py. Every scenario runs on the CPU path in fp32 and,
on a GPU box, through the HIP kernels in fp32 and bf16. Small configurations made here, with sizes that differ
between layers and values that obvious choices would make equal or 1: grouped and single heads, one key head for all,
value sizes unlike key sizes, chunks of 1 position and chunks longer than any prompt, one bucket, one tap, layers
without a feed-forward, either mixer first, head sizes that the matrix-core kernels take and sizes they do not."""
import json
import os

import numpy as np
import pytest
import torch

import lamisun_oracle as oracle
from llmss_amd.engine import LLMEngine, SamplingParams, build_model
from llmss_amd.models.config import ModelConfig
from llmss_amd.models.weights import lamisun_state_dict

gpu = pytest.mark.gpu
RUNS = [pytest.param("cpu", "float32", id="cpu-fp32"), pytest.param("cuda", "float32", marks=gpu, id="gpu-fp32"),
        pytest.param("cuda", "bfloat16", marks=gpu, id="gpu-bf16")]


def lat(heads, dim, rot, vdim, rank, scale, base=10000.0, ff=None, dims=None):
    return dict(type="latent_attention",
                mixer=dict(heads=heads, dim=dim, rot_dim=rot, vdim=vdim, kv_rank=rank, scale=scale,
                           rot=dict(base=base, dims=rot if dims is None else dims)),
                mlp=dict(kind="dense", ff=ff) if ff else None)


def att(heads, kv, dim, vdim, scale, diff, chunk, ff=None):
    return dict(type="attention",
                mixer=dict(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale, diff=diff,
                           mask=dict(size=chunk)),
                mlp=dict(kind="dense", ff=ff) if ff else None)


def model(vocab, width, eps, taps, scale, buckets, mp, mc, layers):
    return dict(architecture="Lamisun", vocab=vocab, width=width, norm=dict(eps=eps), canon=dict(taps=taps),
                embedding=dict(scale=scale, bigram=dict(buckets=buckets, mul_prev=mp, mul_cur=mc)), layers=layers)


CONFIGS = {
    # both mixers alternating, a layer without a feed-forward, grouped heads, chunks that are no multiple of a page
    "mixed": model(97, 40, 1e-5, 4, 0.7, 53, 29, 11, [
        lat(3, 8, 4, 12, 20, 0.3, base=300.0, ff=56),
        att(4, 2, 8, 12, 0.35, 0.2, 10, ff=48),
        lat(2, 16, 8, 6, 12, 0.2),
        att(2, 1, 16, 8, 0.25, 0.4, 7, ff=24),
    ]),
    # attention first and twice in a row; single heads, every head its own key head, a chunk of one position (a row
    # sees itself alone) and a chunk longer than any prompt; one bucket, multipliers of 1, one tap, embedding unscaled
    "plain": model(61, 24, 1e-6, 1, 1.0, 1, 1, 1, [
        att(1, 1, 8, 8, 0.35, 0.1, 1, ff=32),
        att(3, 3, 4, 6, 0.5, 0.3, 1000),
        lat(1, 8, 2, 8, 8, 0.35, base=50.0, ff=16),
    ]),
    # sizes the matrix-core kernels take: key sizes 32, 64, 128; cached latent rows of 64, 128 and 256 numbers
    "wide": model(83, 64, 1e-6, 2, 2.0, 211, 1000003, 7919, [
        lat(4, 32, 16, 32, 48, 0.15, ff=128),
        att(4, 2, 64, 64, 0.125, 0.3, 48, ff=96),
        lat(2, 64, 32, 64, 96, 0.1, base=250.0),
        att(2, 1, 128, 32, 0.09, 0.25, 64, ff=64),
        lat(2, 48, 64, 40, 192, 0.1, ff=64),
        att(8, 2, 32, 24, 0.18, 0.15, 33),
    ]),
    # odd sizes everywhere (no dimension a multiple of 8), rotation of one pair, two taps
    "odd": model(51, 36, 1e-5, 2, 1.3, 7, 5, 3, [
        att(6, 3, 6, 5, 0.4, 0.35, 5, ff=27),
        lat(5, 6, 2, 7, 10, 0.4, base=20.0, ff=19),
        lat(3, 10, 6, 5, 14, 0.3, dims=4),  # the last two numbers of the rotated part do not turn
    ]),
}


class Case:
    def __init__(self, name, tmp, device, dtype, seed=0):
        self.cfg = CONFIGS[name] if name in CONFIGS else BROAD
        mc = ModelConfig.from_hf_dict(self.cfg)
        self.sd = lamisun_state_dict(mc, seed=seed)
        d = tmp / f"{name}-{seed}"
        d.mkdir(exist_ok=True)
        from safetensors.torch import save_file

        save_file({k: v.contiguous() for k, v in self.sd.items()}, str(d / "model.safetensors"))
        (d / "config.json").write_text(json.dumps(self.cfg))
        self.path, self.device, self.dtype = str(d), device, dtype
        self.model = build_model(self.path, dtype=dtype, device=device)
        self.V = self.cfg["vocab"]
        self._ref = {}

    def engine(self, tokens=512, slots=4, block=16, **kw):
        return LLMEngine(self.model, max_num_seqs=slots, block_size=block, num_blocks=-(-tokens // block),
                         max_model_len=tokens, max_batched_tokens=tokens, use_graphs=kw.pop("use_graphs", False),
                         autotune=False, **kw)

    def ref(self, tokens):
        key = tuple(tokens)
        if key not in self._ref:
            self._ref[key] = oracle.forward(self.cfg, self.sd, list(tokens))[0].float()
        return self._ref[key]

    def close(self, got, want, what=""):
        got, want = got.float().cpu(), want.float()
        d = (got - want) - (got - want).mean(-1, keepdim=True)
        err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-3)
        if self.dtype == "float32":
            assert float(err.max()) < 2e-4, f"{what}: relative error {float(err.max()):.3g} at row {int(err.argmax())}"
            return
        # bf16: the difference of two maps, normed afterwards, magnifies rounding now and then (the plain bf16
        # evaluation of the design shows single rows at 0.2 among medians of 0.015), so the typical row is held
        # tightly and the worst one loosely; what a kernel gets wrong shows in the fp32 runs and in the op tests
        assert float(err.median()) < (4e-2 if len(err) >= 8 else 0.12) and float(err.max()) < 0.35, \
            f"{what}: relative error median {float(err.median()):.3g}, max {float(err.max()):.3g} at row {int(err.argmax())}"


def toks(n, V, seed):
    return np.random.default_rng(seed).integers(0, V, n).tolist()


@pytest.fixture(scope="module")
def cases(tmp_path_factory):
    tmp = tmp_path_factory.mktemp("lamisun")
    made = {}

    def get(name, device, dtype):
        k = (name, device, dtype)
        if k not in made:
            made[k] = Case(name, tmp, device, dtype)
        return made[k]
    return get


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_whole_prompt_every_position(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(75, c.V, 1)  # past the edges of every chunk but the longest, and of four pages
    eng = c.engine()
    got = eng.replay_step([(0, t, list(range(len(t))))], end=[0])
    c.close(got, c.ref(t), "whole prompt")
    for n in (1, 2, 3):  # the first tokens of a sequence on their own, in the slot the last request left
        got = eng.replay_step([(n, t[:n], list(range(n)))], end=[n])
        c.close(got, c.ref(t[:n]), f"first {n} token(s)")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_residual_stream_after_every_layer(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(19, c.V, 2)
    want = oracle.forward(c.cfg, c.sd, t)[1]
    seen = {}
    c.model.tap = lambda i, x: seen.__setitem__(i, x.detach().float().cpu().clone())
    try:
        c.engine().replay_step([(0, t, [len(t) - 1])], end=[0])
    finally:
        c.model.tap = None
    assert sorted(seen) == list(range(len(want)))
    tol = 2e-4 if dtype == "float32" else 0.12  # bf16: the plain bf16 evaluation reaches 0.08 behind a two-map layer
    for i, w in enumerate(want):
        rel = (seen[i] - w.float()).abs().max() / w.abs().max()
        assert float(rel) < tol, f"layer {i}: {float(rel):.3g}"


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_prefill_against_token_by_token_decoding(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(40, c.V, 3)
    eng = c.engine()
    rows = [eng.replay_step([(0, [tok], [0])]) for tok in t]  # every token decoded alone, from position 0 on
    eng.replay_step([], end=[0])
    c.close(torch.cat(rows), c.ref(t), "token by token")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", ["mixed", "wide"])
@pytest.mark.parametrize("cuts", [(2, 2, 2, 3, 5, 16, 17, 2, 1, 1, 9), (15, 1, 16, 1, 17, 6), (33, 2, 21),
                                  (1, 2, 70, 2, 33, 1, 1, 30), (9, 1, 10, 10, 1, 19, 2)])
def test_portions_of_several_sizes(cases, cuts, name, device, dtype):
    # portions that end one before, at and one after the edges of chunks (7, 10, 33, 48, 64) and pages (16)
    c = cases(name, device, dtype)
    t = toks(sum(cuts), c.V, 4)
    eng = c.engine()
    got, at = [], 0
    for n in cuts:
        got.append(eng.replay_step([(7, t[at:at + n], list(range(n)))]))
        at += n
    eng.replay_step([], end=[7])
    c.close(torch.cat(got), c.ref(t), f"portions {cuts}")


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", ["mixed", "plain", "wide"])
def test_mixed_batch_of_unequal_requests_equals_each_alone(cases, name, device, dtype):
    c = cases(name, device, dtype)
    seqs = {0: toks(50, c.V, 5), 1: toks(23, c.V, 6), 2: toks(9, c.V, 7), 3: toks(37, c.V, 8)}
    # per step: how many tokens of each request (0 = sits the step out); single tokens ride beside portions
    plan = [{0: 17, 1: 2}, {0: 1, 1: 5, 2: 9}, {0: 1, 1: 16, 3: 30}, {0: 31, 3: 1}, {3: 1, 1: 0}, {3: 5}]
    eng = c.engine(tokens=256)
    at = {k: 0 for k in seqs}
    got = {k: [] for k in seqs}
    for step in plan:
        entries, end = [], []
        for k, n in step.items():
            if n == 0:
                continue
            entries.append((k, seqs[k][at[k]:at[k] + n], list(range(n))))
            at[k] += n
            if at[k] == len(seqs[k]):
                end.append(k)
        out = eng.replay_step(entries, end)
        r = 0
        for k, tk, _ in entries:
            got[k].append(out[r:r + len(tk)])
            r += len(tk)
    assert at == {k: len(v) for k, v in seqs.items()}
    for k, t in seqs.items():
        c.close(torch.cat(got[k]), c.ref(t), f"request {k} in the mixed batch")


@pytest.mark.parametrize("device,dtype", RUNS)
def test_pages_and_state_slots_are_used_again(cases, device, dtype):
    c = cases("mixed", device, dtype)
    eng = c.engine(tokens=64, slots=2, block=16)  # 4 pages, 2 sequences with their state slots
    assert eng.sched.num_free_blocks() == 4
    used = set()
    for r in range(6):  # every round takes the pages and the slots that finished requests gave back
        a, b = toks(30 + r, c.V, 10 + r), toks(17, c.V, 20 + r)
        o1 = eng.replay_step([(2 * r, a[:20], [19]), (2 * r + 1, b, [16])], end=[2 * r + 1])
        used.add(eng.sched.state_slot(2 * r))
        assert eng.sched.num_free_blocks() == 2
        o2 = eng.replay_step([(2 * r, a[20:], list(range(len(a) - 20)))], end=[2 * r])
        assert eng.sched.num_free_blocks() == 4 and eng.sched.num_running() == 0
        c.close(o1, torch.stack([c.ref(a)[19], c.ref(b)[16]]), f"round {r}, first step")
        c.close(o2, c.ref(a)[20:], f"round {r}, second step")
    assert used <= {0, 1}
    with pytest.raises(RuntimeError):  # a third live request has no slot
        eng.replay_step([(100, [1], []), (101, [1], []), (102, [1], [])])
    with pytest.raises(RuntimeError):  # more tokens than the pool has pages for; nothing is taken
        eng.replay_step([(200, [1] * 40, []), (201, [1] * 40, [])])
    assert eng.sched.num_free_blocks() == 4 and eng.sched.num_running() == 0


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", ["mixed", "wide"])
def test_long_decoding_across_pages_and_chunks(cases, name, device, dtype):
    c = cases(name, device, dtype)
    t = toks(150, c.V, 30)
    eng = c.engine()
    got = [eng.replay_step([(0, t[:5], [4])])]
    got += [eng.replay_step([(0, [tok], [0])]) for tok in t[5:]]
    c.close(torch.cat(got), c.ref(t)[4:], "long decoding")


@pytest.mark.parametrize("device,dtype", RUNS)
def test_a_token_far_back_decides_the_logits(cases, device, dtype):
    """The query projections of the latent layers are made four times as large: attention turns sharp, and a key
    that is lost or doubled - the first position, a page's first or last row - changes rows far from it. Prompts
    and single decoded tokens."""
    c = cases("mixed", device, dtype, )
    sd = dict(c.sd)
    for i, L in enumerate(c.cfg["layers"]):
        if L["type"] == "latent_attention":
            sd[f"l{i}.mix.q"] = (sd[f"l{i}.mix.q"].float() * 4).to(torch.bfloat16)
    sharp = Case.__new__(Case)
    sharp.__dict__.update(c.__dict__)
    sharp.sd, sharp._ref = sd, {}
    from llmss_amd.models.weights import _lamisun_finish

    sharp.model = type(c.model)(c.model.cfg, _lamisun_finish(c.model.cfg, lambda n: sd[n].float(), c.device,
                                                             c.model.dtype))
    t = toks(330, c.V, 31)
    eng = sharp.engine()
    want = list(range(0, 300, 37)) + [255, 256, 257, 299]
    got = [eng.replay_step([(0, t[:300], want)])]
    got += [eng.replay_step([(0, [tok], [0])]) for tok in t[300:]]
    sharp.close(torch.cat(got), torch.cat([sharp.ref(t)[want], sharp.ref(t)[300:]]), "sharp attention")
    # the oracle itself: dropping position 0 from the sequence changes the last row by much more than the tolerance
    moved = oracle.forward(sharp.cfg, sd, t[1:])[0][-1].float() - sharp.ref(t)[-1]
    assert float(moved.std() / sharp.ref(t)[-1].std()) > 0.01


@pytest.mark.parametrize("device,dtype", RUNS)
@pytest.mark.parametrize("name", list(CONFIGS))
def test_greedy_generation_through_the_engine(cases, name, device, dtype):
    c = cases(name, device, dtype)
    prompts = [toks(11, c.V, 40), toks(3, c.V, 41), toks(26, c.V, 42)]
    eng = LLMEngine(c.model, max_num_seqs=4, block_size=16, num_blocks=32, max_model_len=128, max_batched_tokens=24,
                    prefill_chunk=7, autotune=False)  # its own scheduler cuts the prompts and batches the decodes
    out = eng.generate(prompts, SamplingParams(max_new_tokens=12, is_greedy=True, ignore_eos=True))
    for p, o in zip(prompts, out):
        want = oracle.greedy(c.cfg, c.sd, p, 12)
        if dtype == "float32":
            assert o == want
        else:  # bf16 may flip a near-tie; the tokens before the first difference must then be a true near-tie
            k = next((i for i, (x, y) in enumerate(zip(o, want)) if x != y), None)
            if k is not None:
                lg = oracle.forward(c.cfg, c.sd, p + want[:k])[0][-1]
                assert float(lg[want[k]] - lg[o[k]]) < 0.05 * float(lg.std())


@pytest.mark.parametrize("device,dtype", RUNS)
def test_preempted_requests_start_over_from_an_empty_state(cases, device, dtype):
    """A pool too small for all requests: the scheduler preempts (pages and state slot go back) and recomputes."""
    c = cases("mixed", device, dtype)
    prompts = [toks(20, c.V, 80), toks(18, c.V, 81), toks(22, c.V, 82)]
    eng = LLMEngine(c.model, max_num_seqs=3, block_size=8, num_blocks=9, max_model_len=64, max_batched_tokens=32,
                    autotune=False)
    out = eng.generate(prompts, SamplingParams(max_new_tokens=14, is_greedy=True, ignore_eos=True))
    assert eng.stats["preemptions"] > 0
    if dtype == "float32":
        for p, o in zip(prompts, out):
            assert o == oracle.greedy(c.cfg, c.sd, p, 14)


def test_config_reader_rejects_what_the_design_does_not_have():
    bad = json.loads(json.dumps(CONFIGS["plain"]))
    bad["layers"][0]["type"] = "convolution"
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["mixed"]))
    bad["layers"][1]["mixer"]["kv_heads"] = 3  # does not divide the heads
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["mixed"]))
    bad["layers"][0]["mixer"]["rot"]["dims"] = 6  # more rotated dimensions than the rotated part holds
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["plain"]))
    bad["layers"][0]["mlp"]["kind"] = "moe"
    with pytest.raises(ValueError):
        ModelConfig.from_hf_dict(bad)


def test_config_reader_takes_every_size_and_constant_from_the_file():
    mc = ModelConfig.from_hf_dict(CONFIGS["mixed"])
    assert (mc.model_type, mc.vocab_size, mc.hidden_size, mc.canon_taps, mc.embedding_scale) == \
        ("lamisun", 97, 40, 4, 0.7)
    assert (mc.bigram.buckets, mc.bigram.mul_prev, mc.bigram.mul_cur) == (53, 29, 11)
    a, b = mc.layer_specs[0].mixer, mc.layer_specs[1].mixer
    assert (a.kind, a.heads, a.dim, a.rot_dim, a.vdim, a.kv_rank, a.scale, a.rot.base, a.gate) == \
        ("latent_attention", 3, 8, 4, 12, 20, 0.3, 300.0, True)
    assert (b.kind, b.heads, b.kv_heads, b.dim, b.vdim, b.scale, b.diff, b.chunk) == \
        ("attention", 4, 2, 8, 12, 0.35, 0.2, 10)
    assert mc.layer_specs[2].mlp is None and mc.layer_specs[3].mlp.ff == 24 and not mc.layer_specs[3].mlp.gated
    from llmss_amd.models.weights import lamisun_shapes

    assert mc.num_params() == sum(int(np.prod(s)) for s in lamisun_shapes(mc).values())


def test_loader_checks_shapes_against_the_config(cases, tmp_path):
    c = cases("plain", "cpu", "float32")
    cfg = json.loads(json.dumps(c.cfg))
    cfg["layers"][1]["mixer"]["vdim"] = 12
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    os.symlink(os.path.join(c.path, "model.safetensors"), tmp_path / "model.safetensors")
    with pytest.raises(ValueError):
        build_model(str(tmp_path), dtype="float32", device="cpu")


def test_cache_holds_latent_rows_key_value_pages_and_per_sequence_state(cases):
    c = cases("mixed", "cpu", "float32")
    kv = c.model.allocate_kv_cache(4, 16, num_slots=3)
    assert kv[0][0].shape == (4, 16, 20 + 4) and kv[0][1] is None  # latent row and the rotated key part
    assert kv[1][0].shape == (4, 16, 2 * 2 * 8) and kv[1][1].shape == (4, 16, 2 * 12)  # two maps per key head
    assert c.model.canon_tail.shape == (8, 3, 3, 40)  # mixer and feed-forward of four layers, three inputs back
    assert c.model.prev_token.shape == (3,)
    assert c.model.kv_bytes_per_block(16) == 16 * 4 * ((20 + 4) + (12 + 8) + 2 * (2 * 8 + 12) + (2 * 16 + 8))
    assert c.model.needs_state and c.model.state_bytes_per_slot() == 8 + 4 * 3 * 40 * 8


def test_trace_runner_replays_steps_on_the_cpu_path(cases, tmp_path):
    import subprocess
    import sys

    c = cases("plain", "cpu", "float32")
    t = toks(21, c.V, 50)
    steps = [dict(step=0, entries=[dict(id="a", tokens=t[:9], want=[0, 8])], end=[]),
             dict(step=1, entries=[dict(id="b", tokens=t[:2], want=[])], end=[]),
             dict(step=2, entries=[dict(id="a", tokens=t[9:], want=[11]), dict(id="b", tokens=t[2:3], want=[0])],
                  end=["a", "b"])]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", c.path, "--dtype", "float32",
                        "--out", str(tmp_path), "--max-tokens", "64", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == ["done 0", "done 1", "done 2"]
    g0 = torch.from_numpy(np.fromfile(tmp_path / "0.f32", dtype="<f4").reshape(2, c.V))
    g2 = torch.from_numpy(np.fromfile(tmp_path / "2.f32", dtype="<f4").reshape(2, c.V))
    c.close(g0, c.ref(t)[[0, 8]], "step 0")
    c.close(g2, torch.stack([c.ref(t)[20], c.ref(t[:3])[2]]), "step 2")


# A wider model than the others here, for the GPU: rows of hundreds of tokens through the matrix-core kernels
# (cached latent rows of 64 and 192 numbers, key sizes 32 and 64), several row blocks per portion.
BROAD = model(700, 320, 1e-5, 2, 1.5, 257, 97, 5, [
    lat(5, 48, 16, 48, 48, 0.12, base=5000.0, ff=640),
    lat(10, 32, 32, 32, 160, 0.12, base=5000.0, ff=640),
    att(10, 5, 32, 32, 0.18, 0.4, 50, ff=640),
    att(5, 1, 64, 64, 0.125, 0.1, 512, ff=640),
])


@gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_runner_replays_long_requests_on_the_gpu(cases, tmp_path, dtype):
    """bin/trace_run as a user runs it, on the GPU in both precisions: a request of 600 tokens alone in portions of
    changing size and then token by token, then - in the pages and the slot it gave back - three requests side by
    side, portions of some beside single tokens of others. Every position's logits against the float64 definition."""
    import subprocess
    import sys

    c = cases("broad", "cuda", dtype)
    reqs = {"a": toks(600, c.V, 31), "b": toks(290, c.V, 32), "c": toks(130, c.V, 33), "d": toks(5, c.V, 34)}
    steps, at = [], {k: 0 for k in reqs}

    def feed(pairs):
        ent = []
        for k, n in pairs:
            ent.append(dict(id=k, tokens=reqs[k][at[k]:at[k] + n], want=list(range(n))))
            at[k] += n
        steps.append(dict(step=len(steps), entries=ent, end=[k for k, _ in pairs if at[k] == len(reqs[k])], rows=[
            (k, at[k] - n + j) for k, n in pairs for j in range(n)]))

    cuts = [100, 2, 133, 3, 33, 2, 17, 78, 64, 1, 1, 1, 37]
    i = 0
    while at["a"] < len(reqs["a"]):
        left = len(reqs["a"]) - at["a"]
        feed([("a", min(left, cuts[i % len(cuts)]) if left > 20 else 1)])
        i += 1
    pat = {"b": [150, 1, 90, 1, 1, 2], "c": [2, 1, 1, 30, 1], "d": [1, 1, 3]}
    i = 0
    while any(at[k] < len(reqs[k]) for k in pat):
        pairs = [(k, min(len(reqs[k]) - at[k], pat[k][i % len(pat[k])])) for k in pat
                 if at[k] < len(reqs[k]) and (i + ord(k)) % 5 != 4]
        if pairs:
            feed(pairs)
        i += 1
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", c.path, "--dtype", dtype,
                        "--out", str(tmp_path), "--max-tokens", "640"],
                       input="".join(json.dumps({k: v for k, v in s.items() if k != "rows"}) + "\n" for s in steps),
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert sum(ln.startswith("done") for ln in r.stdout.splitlines()) == len(steps)
    ref = {k: c.ref(v).double() for k, v in reqs.items()}
    every = torch.cat(list(ref.values()))
    spread = float((every - every.mean(-1, keepdim=True)).pow(2).mean().sqrt())
    errs = []
    for s in steps:
        got = torch.from_numpy(np.fromfile(tmp_path / f"{s['step']}.f32", dtype="<f4").reshape(-1, c.V)).double()
        want = torch.stack([ref[k][p] for k, p in s["rows"]])
        d = (got - want) - (got - want).mean(-1, keepdim=True)
        errs.append(d.pow(2).mean(-1).sqrt() / spread)
    errs = torch.cat(errs)
    if dtype == "float32":
        assert float(errs.max()) < 5e-5, f"row {int(errs.argmax())}: {float(errs.max()):.3g} of the logits' spread"
    else:  # bf16 products and activations: the model's own rounding noise (median 0.011, largest 0.022 of the spread)
        assert float(errs.median()) < 0.02 and float(errs.max()) < 0.05, (float(errs.median()), float(errs.max()))


def test_registry_facade_runs_the_design(cases):
    """MODEL_REGISTRY["lamisun"](config, weights): HF-style calls with a growing paged past and a state slot."""
    from llmss_amd.models.registry import MODEL_REGISTRY, Weights
    from llmss_amd.utils.checkpoint import weight_files

    c = cases("mixed", "cpu", "float32")
    cfg = ModelConfig.from_pretrained(c.path)
    lm = MODEL_REGISTRY[cfg.model_type](cfg, Weights(weight_files(c.path), "cpu", torch.float32), max_blocks=16)
    t = toks(21, c.V, 60)
    out = lm(torch.tensor([t[:13]]), use_cache=True)
    c.close(out.logits[0], c.ref(t[:13]), "prompt through the facade")
    out2 = lm(torch.tensor([t[13:]]), past_key_values=out.past_key_values, use_cache=True)
    c.close(out2.logits[0], c.ref(t)[13:], "continuation through the facade")
    lm.release(out2.past_key_values)
    assert len(lm._free_state) == 16


def test_preset_builds_and_steps():
    m = build_model("tiny-lamisun", dtype="float32", device="cpu")
    eng = LLMEngine(m, max_num_seqs=2, block_size=16, num_blocks=8, max_model_len=64, max_batched_tokens=64,
                    autotune=False)
    out = eng.generate([[1, 2, 3]], SamplingParams(max_new_tokens=4, is_greedy=True, ignore_eos=True))
    assert len(out[0]) == 4


@gpu
def test_decode_graphs_and_autotuned_projections_decode_right(cases):
    """Serving defaults on a GPU: GEMM plans timed per decode bucket, decode steps replayed from captured graphs
    (state slots ride in the graphs' static buffers), pipelined decode."""
    c = cases("wide", "cuda", "bfloat16")
    assert c.model.gemm_shapes()
    eng = LLMEngine(c.model, max_num_seqs=4, block_size=16, num_blocks=32, max_model_len=96, max_batched_tokens=64)
    assert eng.graphs
    prompts = [toks(9, c.V, 70), toks(17, c.V, 71), toks(2, c.V, 72)]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=10, is_greedy=True, ignore_eos=True))
    for p, out in zip(prompts, outs):
        want = oracle.greedy(c.cfg, c.sd, p, 10)
        k = next((i for i, (x, y) in enumerate(zip(out, want)) if x != y), None)
        if k is not None:
            lg = oracle.forward(c.cfg, c.sd, p + want[:k])[0][-1]
            assert float(lg[want[k]] - lg[out[k]]) < 0.05 * float(lg.std())


@gpu
def test_fp32_decode_graphs_reproduce_the_oracle_exactly(cases):
    c = cases("mixed", "cuda", "float32")
    eng = LLMEngine(c.model, max_num_seqs=4, block_size=16, num_blocks=32, max_model_len=96, max_batched_tokens=64,
                    autotune=False)
    assert eng.graphs
    prompts = [toks(9, c.V, 73), toks(30, c.V, 74), toks(1, c.V, 75)]
    outs = eng.generate(prompts, SamplingParams(max_new_tokens=20, is_greedy=True, ignore_eos=True))
    for p, out in zip(prompts, outs):
        assert out == oracle.greedy(c.cfg, c.sd, p, 20)
