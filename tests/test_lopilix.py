"""Lopilix through the framework (config registry, weight images, sequence state cache, step
scheduler, kernels) against the plain float64 oracle in ``lopilix_oracle.py``.

Every test runs on the CPU backend (plain PyTorch ops) and, marked ``gpu``, on the HIP kernels.  The
models are tiny and random; fp32 matrix products make the comparison sharp (a key one place off, a
lost recurrent state, a pass of a looped layer that reads another pass's keys, a wrong page or a
forgotten stream coefficient shows as an error thousands of times the tolerance), and some tests run
the bf16 mode.  Where random weights would hide a fault, the weights are set so that one key dominates."""
import json
import math
import os
import pickle
import subprocess
import sys

import numpy as np
import pytest
import torch

import lopilix_oracle as oracle
import lopilix_util as lu
from conftest import gpu_available
from flexible_llm_sharding_amd.runtime.batch import StepEntry
from flexible_llm_sharding_amd.serve import generate, load_runner

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
TOL = 2e-4          # fp32 products against float64, relative to a logit row's spread
F = torch.float64


@pytest.fixture(autouse=True)
def _need_gpu(request):
    params = getattr(getattr(request.node, "callspec", None), "params", {})
    if "cuda" in str(params.get("device", "")) and not gpu_available():
        pytest.skip("no GPU")


def build(tmp_path, layers, seed=0, dtype=torch.float32, device="cpu", **kw):
    cfg = lu.config(layers, **{k: v for k, v in kw.items() if k in ("width", "vocab", "eps", "mult", "streams", "logit_scale", "loop",
                                                                     "max_positions")})
    sd = lu.random_weights(cfg, seed, **({"std": kw["std"]} if "std" in kw else {}))
    path = lu.write_model(str(tmp_path / f"m{seed}"), cfg, sd)
    runner = load_runner(path, dtype, device, max_tokens=kw.get("max_tokens", 64), max_seqs=kw.get("max_seqs", 2),
                         layer_num_per_shard=kw.get("lnps"), token_budget=kw.get("token_budget", 16384),
                         resident=kw.get("resident", True))
    return cfg, sd, runner, path


def run_cut(runner, rid, toks, cuts, end=True):
    """Feed ``toks`` in portions of the sizes ``cuts`` (the rest one by one) -> logits of every position."""
    out, at = [], 0
    sizes = list(cuts) + [1] * (len(toks) - sum(cuts))
    for n in sizes:
        last = at + n == len(toks)
        r = runner.step([StepEntry(rid, toks[at:at + n], range(n))], [rid] if (last and end) else [])
        out.append(r[0][0])
        at += n
    return np.concatenate(out, 0)


# differential attention + dense, HGRN2 + experts, latent attention + experts without groups, HGRN2 without a
# feed-forward, a multi-head differential attention whose whole head is rotated; layers 1 .. 3 run twice
STACK = [(lu.attn(), lu.dense()),
         (lu.hgrn(), lu.moe()),
         (lu.latent(), lu.moe(experts=5, top=3, ff=9, groups=None, scale=0.8)),
         (lu.hgrn(heads=2, dim=20, vdim=6), None),
         (lu.attn(heads=3, kv_heads=3, dim=8, vdim=5, rot_dims=8, base=1000.0, scale=0.7, diff=0.6), lu.moe(experts=4, top=4, ff=10, groups=(2, 2)))]
LOOP = (1, 4, 2)


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,layers,kw", [
    ("differential-attention", [(lu.attn(scale=1.5), None)], {}),
    ("differential-attention-one-head-no-rotation", [(lu.attn(heads=1, kv_heads=1, dim=4, vdim=3, rot_dims=0), None)], {}),
    ("differential-attention-multi-head-full-rotation", [(lu.attn(heads=3, kv_heads=3, dim=8, vdim=8, rot_dims=8), None)], {}),
    ("differential-attention-rescaled-rotation", [(lu.attn(scaling=lu.SCALING), None)], {}),
    ("hgrn2", [(lu.hgrn(), None)], {}),
    ("hgrn2-one-head-wide-state", [(lu.hgrn(heads=1, dim=37, vdim=70), None)], {}),
    ("hgrn2-narrow", [(lu.hgrn(heads=5, dim=1, vdim=1), None)], {}),
    ("latent-attention", [(lu.latent(), None)], {}),
    ("latent-attention-unscaled-rotation", [(lu.latent(scaling=None, heads=1, kv_rank=3, vdim=12), None)], {}),
    ("latent-attention-every-pair-slowed", [(lu.latent(scaling={"factor": 2.0, "original": 8, "fast": 64.0, "slow": 32.0}), None)], {}),
    ("dense-feed-forward", [(lu.hgrn(), lu.dense(ff=33))], {}),
    ("experts-grouped", [(lu.hgrn(), lu.moe(experts=12, top=3, groups=(4, 2)))], {}),
    ("experts-groups-of-one", [(lu.hgrn(), lu.moe(experts=5, top=2, groups=(5, 3)))], {}),
    ("experts-all-groups-kept-all-chosen", [(lu.hgrn(), lu.moe(experts=4, top=4, groups=(2, 2), scale=1.0))], {}),
    ("experts-top-1-no-groups", [(lu.hgrn(), lu.moe(experts=7, top=1, groups=None))], {}),
    ("one-stream", [(lu.attn(), lu.dense()), (lu.hgrn(), lu.moe())], {"streams": 1}),
    ("five-streams", [(lu.attn(), lu.dense()), (lu.latent(), None)], {"streams": 5}),
    ("unit-multipliers", [(lu.attn(), lu.moe())], {"mult": 1.0, "logit_scale": 1.0}),
    ("loop-of-one-layer-three-times", [(lu.attn(), None), (lu.hgrn(), lu.dense()), (lu.latent(), None)], {"loop": (1, 2, 3)}),
    ("loop-once", [(lu.attn(), None), (lu.hgrn(), lu.dense())], {"loop": (0, 2, 1)}),
    ("width-not-a-multiple-of-four", [(lu.attn(), lu.moe()), (lu.latent(), lu.dense())], {"width": 34}),
])
def test_mechanism_alone(tmp_path, device, name, layers, kw):
    cfg, sd, runner, _ = build(tmp_path, layers, seed=3, device=device, **kw)
    toks = lu.tokens(45, cfg["vocab"], 1)
    want = lu.oracle_logits(cfg, sd, toks)
    assert lu.rel_err(run_cut(runner, "a", toks, [len(toks)]), want) < TOL
    assert lu.rel_err(run_cut(runner, "b", toks, [30, 2]), want) < TOL
    runner.close()


def test_oracle_parts_agree_with_their_definitions():
    """The oracle's own pieces on hand-made inputs: both pair layouts of the rotation, the rescaled
    frequencies and their amplitude, the recurrence by hand, routing among groups, lambda, the layer order."""
    x = torch.tensor([[[0.0, 0.0, 5.0, 6.0, 7.0]], [[1.0, 0.0, 0.0, 2.0, 7.0]]], dtype=F)
    r = oracle.rotate(x, {"dims": 2, "base": 100.0}, "pairs")
    assert torch.allclose(r[1, 0], torch.tensor([math.cos(1.0), math.sin(1.0), 0.0, 2.0, 7.0], dtype=F))
    r = oracle.rotate(x, {"dims": 4, "base": 100.0}, "half")           # pairs (0, 2) and (1, 3); f = 1, 0.1
    assert torch.allclose(r[1, 0], torch.tensor([math.cos(1.0), -2 * math.sin(0.1), math.sin(1.0), 2 * math.cos(0.1), 7.0], dtype=F))
    assert torch.equal(r[0], x[0])
    rot = {"dims": 16, "base": 100.0, "scaling": {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 1.0}}
    f, amp = oracle.rot_freqs(rot)
    f0, one = oracle.rot_freqs({"dims": 16, "base": 100.0})
    ratio = [a / b for a, b in zip(f, f0)]
    assert one == 1.0 and abs(amp - (0.1 * math.log(8.0) + 1.0)) < 1e-15
    # entry numbers where a pair turns 4 times and once over 64 positions: 16 ln(64 / (2 pi t)) / (2 ln 100)
    lo, hi = math.floor(16 * math.log(64 / (8 * math.pi)) / (2 * math.log(100))), math.ceil(16 * math.log(64 / (2 * math.pi)) / (2 * math.log(100)))
    assert (lo, hi) == (1, 5)
    assert ratio[0] == 1.0 and ratio[1] == 1.0 and abs(ratio[3] - (1 - 0.5 + 0.5 / 8)) < 1e-12 and all(abs(q - 1 / 8) < 1e-12 for q in ratio[5:])
    # the recurrence with one head, one state row and gate 1/2: S = S / 2 + v / 2
    sd = {"q": torch.tensor([[100.0]], dtype=F), "f": torch.zeros(1, 1, dtype=F), "f.b": torch.zeros(1, dtype=F), "lower": torch.zeros(1, dtype=F),
          "v": torch.tensor([[1.0], [0.0]], dtype=F), "norm": torch.ones(2, dtype=F), "o": torch.eye(2, dtype=F)}
    h = torch.tensor([[1.0], [1.0], [1.0]], dtype=F)
    S = torch.zeros(2, dtype=F)
    rows = []
    for t in range(3):
        S = 0.5 * S + 0.5 * torch.tensor([1.0, 0.0], dtype=F)
        rows.append(oracle.rms(S * 100.0, 1e-6))
    assert torch.allclose(oracle.hgrn2(sd, "", {"heads": 1, "dim": 1, "vdim": 2}, h, 1e-6), torch.stack(rows), atol=1e-9)
    # a lower bound of 1 never forgets and never writes
    sd["lower"] = torch.ones(1, dtype=F)
    assert oracle.hgrn2(sd, "", {"heads": 1, "dim": 1, "vdim": 2}, h, 1e-6).abs().max() == 0.0
    # groups (0,1) (2,3) (4,5): worth 0.9+0.1, 0.6+0.6, 0.7+0.2 -> groups 1 and 0 compete, expert 4 does not
    logit = lambda p: math.log(p / (1 - p))
    z = torch.tensor([logit(p) for p in (0.9, 0.1, 0.6, 0.6, 0.7, 0.2)], dtype=F)
    got = oracle.route(z, {"experts": 6, "top": 3, "scale": 2.0, "groups": {"count": 3, "keep": 2}})
    assert [e for e, _ in got] == [0, 2, 3] and np.allclose([w for _, w in got], [2 * 0.9 / 2.1, 2 * 0.6 / 2.1, 2 * 0.6 / 2.1])
    got = oracle.route(z, {"experts": 6, "top": 3, "scale": 1.0})
    assert [e for e, _ in got] == [0, 4, 2]
    lam = oracle.diff_lambda({"lq1": torch.tensor([1.0, 2.0], dtype=F), "lk1": torch.tensor([0.5, 0.25], dtype=F),
                              "lq2": torch.zeros(2, dtype=F), "lk2": torch.ones(2, dtype=F)}, "", 0.2)
    assert abs(lam - (math.e - 1.0 + 0.2)) < 1e-12
    assert oracle.layer_order({"layers": [0] * 5, "loop": {"start": 1, "stop": 3, "times": 3}}) == [0, 1, 2, 1, 2, 1, 2, 3, 4]
    assert oracle.layer_order({"layers": [0] * 2}) == [0, 1]


# ----------------------------------------------- prompts, portions, decoding, first tokens
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_portions_and_decode(tmp_path, device):
    """The same sequence whole, token by token, and in portions of 2, 3, 7, 16 and 17 tokens: keys, latent
    rows and recurrent states of both passes of the looped layers all cross the cuts."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=5, device=device, loop=LOOP)
    toks = lu.tokens(50, cfg["vocab"], 2)
    want = lu.oracle_logits(cfg, sd, toks)
    for cuts in ([50], [], [2, 2, 3, 7, 16, 17], [17, 16, 2], [1, 2, 40]):
        assert lu.rel_err(run_cut(runner, "r", toks, cuts), want) < TOL, cuts
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_residual_streams_after_every_layer_run(tmp_path, device):
    """What leaves every layer run (a looped layer counts each time) against the oracle's summed streams,
    through the layer functions on the runner's own weights and cache."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=4, device=device, loop=LOOP)
    toks = lu.tokens(21, cfg["vocab"], 8)
    trace = []
    lu.oracle_logits(cfg, sd, toks, trace)
    from flexible_llm_sharding_amd.runtime.batch import pack_step
    batch = pack_step([StepEntry("t", toks, [len(toks) - 1])], runner.seq_cache)
    meta = batch.device_tensors(runner.dev)
    W = {}
    for k in range(len(runner.my_shards)):
        W.update(runner.prefetcher.acquire(k))
    state, n = None, 0
    for name in runner.names:
        state = runner.family.run_layer(runner.ctx, name, W[name], state, batch, meta)
        if name[0] == "l":
            got = state.float().reshape(len(toks), cfg["streams"], cfg["width"]).sum(1).cpu().double()
            assert (got - trace[n]).abs().max() < 1e-4 * trace[n].abs().max(), name
            n += 1
    assert n == len(trace) == 8
    runner.seq_cache.release("t")
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_over_pages(tmp_path, device):
    """A short prompt, then 120 decoded tokens: pages of 16 fill one after the other, the recurrent states
    are carried 120 times, and nothing is ever given back while the request lives (every key stays visible)."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=6, device=device, loop=LOOP)
    toks = lu.tokens(125, cfg["vocab"], 7)
    got = run_cut(runner, "r", toks, [5], end=False)
    assert lu.rel_err(got, lu.oracle_logits(cfg, sd, toks)) < TOL
    cache = runner.seq_cache
    assert cache.pages_trimmed == 0 and all(p >= 0 for p in cache.requests["r"].pages) and len(cache.requests["r"].pages) == 8
    cache.release("r")
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    """Sequences of one, two and three tokens, whole and decoded."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=8, device=device, loop=LOOP)
    for n in (1, 2, 3):
        toks = lu.tokens(n, cfg["vocab"], 20 + n)
        want = lu.oracle_logits(cfg, sd, toks)
        assert lu.rel_err(run_cut(runner, "w", toks, [n]), want) < TOL
        assert lu.rel_err(run_cut(runner, "d", toks, []), want) < TOL
    runner.close()


# ------------------------------------------------------------ batches, pages and slots
@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone(tmp_path, device):
    """Requests of 1, 9, 33 and 50 tokens in one step, then decoded together while the short ones
    finish first; also cut into two micro-batches by a small token budget."""
    for budget in (16384, 40):
        cfg, sd, runner, _ = build(tmp_path, STACK, seed=9, device=device, token_budget=budget, loop=LOOP)
        lens, extra = [1, 9, 33, 50], [3, 12, 0, 6]
        seqs = [lu.tokens(n + e, cfg["vocab"], 30 + i) for i, (n, e) in enumerate(zip(lens, extra))]
        want = [lu.oracle_logits(cfg, sd, s) for s in seqs]
        got = [[] for _ in seqs]
        live = list(range(4))
        res = runner.step([StepEntry(i, seqs[i][:lens[i]], range(lens[i])) for i in live], [i for i in live if extra[i] == 0])
        for i, r in zip(live, res):
            got[i].append(r[0])
        for t in range(max(extra)):
            live = [i for i in range(4) if extra[i] > t]
            res = runner.step([StepEntry(i, [seqs[i][lens[i] + t]], [0]) for i in live], [i for i in live if extra[i] == t + 1])
            for i, r in zip(live, res):
                got[i].append(r[0])
        for i in range(4):
            assert lu.rel_err(np.concatenate(got[i], 0), want[i]) < TOL, (budget, i)
        assert not runner.seq_cache.requests
        runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_used_again(tmp_path, device):
    """Requests come and go through pools of two slots and a few pages: whoever inherits a page or a
    slot (with the last owner's keys, latent rows and recurrent states still in it) computes what it
    computes alone, and pools that run out grow without disturbing the live request."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=11, device=device, max_tokens=40, max_seqs=2, loop=LOOP)
    cache = runner.seq_cache
    a, b, c = (lu.tokens(n, cfg["vocab"], 40 + n) for n in (37, 22, 41))
    wa, wb, wc = (lu.oracle_logits(cfg, sd, s) for s in (a, b, c))
    assert lu.rel_err(run_cut(runner, "a", a, [30]), wa) < TOL
    ga = run_cut(runner, "a2", a, [10, 2], end=False)                       # stays alive
    gb = run_cut(runner, "b", b, [22])                                      # inherits a's first slot
    assert cache.slots_reused > 0 and cache.pages_reused > 0
    gc = run_cut(runner, "c", c, [3, 30])
    n0 = cache.n_slots
    others = [run_cut(runner, f"x{i}", b, [5], end=False) for i in range(3)]    # more requests than slots
    assert cache.n_slots > n0
    tail = runner.step([StepEntry("a2", [a[0]], [0])], ["a2"])[0][0]         # a2's state survived the growth
    assert lu.rel_err(tail, lu.oracle_logits(cfg, sd, a + [a[0]])[-1:]) < TOL
    for g, w in ((ga, wa), (gb, wb), (gc, wc)) + tuple((o, wb) for o in others):
        assert lu.rel_err(g, w) < TOL
    runner.close()


# ----------------------------------------------------- shards, bf16, generation
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("lnps", [1, 3])
def test_few_layers_per_shard_stream_weights(tmp_path, device, lnps):
    """Weights streamed shard by shard: the passes of a looped layer land in different shards (its image is
    loaded again) or in one (loaded once, shared)."""
    cfg = lu.config(STACK, loop=LOOP)
    sd = lu.random_weights(cfg, 13)
    path = lu.write_model(str(tmp_path / "s"), cfg, sd)
    runner = load_runner(path, torch.float32, device, max_tokens=64, layer_num_per_shard=lnps, resident=False)
    toks = lu.tokens(40, cfg["vocab"], 3)
    assert lu.rel_err(run_cut(runner, "r", toks, [20, 2]), lu.oracle_logits(cfg, sd, toks)) < TOL
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_products_stay_close(tmp_path, device):
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=14, device=device, dtype=torch.bfloat16, loop=LOOP)
    toks = lu.tokens(40, cfg["vocab"], 4)
    want = lu.oracle_logits(cfg, sd, toks)
    whole, cut = run_cut(runner, "a", toks, [40]), run_cut(runner, "b", toks, [9, 2])
    assert lu.rel_err(whole, want) < 0.15 and lu.rel_err(cut, want) < 0.15      # (the worst row)
    assert lu.rel_err(cut, whole) < 0.12
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_head_sizes_of_the_matrix_core_kernels(tmp_path, device):
    """bf16 with head sizes that the matrix-core prompt attention serves on the GPU (differential attention
    with keys of 64 and values of 128; latent attention with 64 + 64 wide keys made per head from the step's
    rows, and a latent of 128 + 64 that the heads-as-columns decode kernel reads): a prompt of several row
    tiles, a portion that continues it, then decoding.  Whole-prompt and decoded logits both stay within
    bf16 rounding of the oracle, and of each other."""
    layers = [(lu.attn(heads=4, kv_heads=2, dim=64, vdim=128, rot_dims=32, base=1e4, scale=0.12), lu.moe()),
              (lu.latent(heads=4, dim=64, rot_dim=64, vdim=128, kv_rank=128, base=1e4, scale=0.09), None),
              (lu.attn(heads=2, kv_heads=1, dim=128, vdim=64, rot_dims=128, base=1e4, scale=0.09), lu.dense())]
    cfg, sd, runner, _ = build(tmp_path, layers, seed=23, device=device, dtype=torch.bfloat16, max_tokens=512, std=0.2)
    toks = lu.tokens(230, cfg["vocab"], 6)
    want = lu.oracle_logits(cfg, sd, toks)
    whole = run_cut(runner, "a", toks, [230])
    cut = run_cut(runner, "b", toks, [150, 40])
    # (the difference of two attention maps, divided by its own root mean square, amplifies the rounding of both where
    # the maps nearly cancel: a few rows stand far above the rest, so the bound is on the mean and on nine rows in ten)
    for got, ref, mean, q90 in ((whole, want, 0.05, 0.08), (cut, want, 0.05, 0.08), (cut, whole, 0.05, 0.08)):
        e = lu.row_errs(got, ref)
        assert e.mean() < mean and np.quantile(e, 0.9) < q90, (e.mean(), np.quantile(e, 0.9))
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """serve.generate: prompts of unequal length, 12 new tokens each; the tokens are the oracle's
    greedy continuation (recomputed from scratch at every step)."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=15, device=device, loop=LOOP)
    prompts = [lu.tokens(n, cfg["vocab"], 50 + n) for n in (3, 17, 26)]
    got = generate(runner, prompts, 12)
    for p, g in zip(prompts, got):
        seq = list(p)
        for t in g:
            z = lu.oracle_logits(cfg, sd, seq)[-1]
            top2 = np.sort(z)[-2:]
            if top2[1] - top2[0] > 1e-3:              # (a tie within rounding may go either way)
                assert t == int(z.argmax())
            seq.append(t)
    assert not runner.seq_cache.requests
    runner.close()


# ------------------------------------------- one token that stands out, far back and at page borders
def _marked_model(tmp_path, kind):
    """One layer whose weights make one marked token decide every later row.  Channel 0 of the embedding is
    the same for every token, channel 1 is zero except for the marked token, where it is large; positions
    add next to nothing.  ``attention``: every query of map 1 points along u, every key along -u, the marked
    token's along +u, so after the per-head norms its score is +scale * dim against -scale * dim for all
    others, however many hundreds there are.  ``latent``: the latent's first entry carries that sign, W_uk
    turns it into +-u, the unrotated query is u.  ``hgrn2``: lower bounds next to 1 keep what the marked
    token wrote (a large value) for hundreds of steps."""
    D, vocab, mark, d = 24, 40, 7, 8
    u = torch.tensor([0.0, 0.0, 1.0, -1.0, 1.0, 1.0, -1.0, 1.0])            # (entries 0, 1 are a rotated pair: left out)
    mixer = {"attention": lu.attn(heads=2, kv_heads=1, dim=d, vdim=6, rot_dims=2, base=1e6, scale=1.6, diff=0.35),
             "latent": lu.latent(heads=2, dim=d, rot_dim=4, vdim=6, kv_rank=5, base=1e6, scaling=None, scale=0.4),
             "hgrn2": lu.hgrn(heads=2, dim=4, vdim=6)}[kind]
    cfg = lu.config([(mixer, None)], width=D, vocab=vocab, mult=1.0, streams=2, logit_scale=1.0, max_positions=320)
    sd = {k: v.float() for k, v in lu.random_weights(cfg, 12, std=0.05).items()}
    sd["embed"] *= 0.05
    sd["pos"] *= 0.02
    sd["embed"][:, 0] = 4.0
    sd["embed"][:, 1] = 0.0
    sd["embed"][mark, 1] = 12.0
    sd["l0.norm1"][:] = 1.0
    x = "l0.mix."
    if kind == "attention":
        sd[x + "q.norm"][:] = 1.0
        sd[x + "k.norm"][:] = 1.0
        for hh in range(2):
            sd[x + "q"][hh * 2 * d:hh * 2 * d + d, 0] = u                   # map 1 of head hh
        sd[x + "k"][:d, 0] = -u
        sd[x + "k"][:d, 1] = u
        sd[x + "v"][:, 1] = 3.0
    elif kind == "latent":
        sd[x + "dkv.norm"][:] = 1.0
        sd[x + "dkv"][0, 0], sd[x + "dkv"][0, 1] = -1.0, 1.0
        for hh in range(2):
            sd[x + "q"][hh * (d + 4):hh * (d + 4) + d, 0] = u
            sd[x + "uk"][hh * d:(hh + 1) * d, 0] = u / math.sqrt(5.0)
        sd[x + "uv"][:, 0] = 3.0 / math.sqrt(5.0)
    else:
        sd[x + "lower"][:] = 0.996
        sd[x + "q"][:, 0] = 1.0
        sd[x + "v"][:, 1] = 3.0
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    return cfg, sd, lu.write_model(str(tmp_path / f"mark_{kind}"), cfg, sd), mark, vocab


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("kind", ["attention", "latent", "hgrn2"])
def test_one_token_stands_out_far_back_and_at_page_borders(tmp_path, device, kind):
    """The marked token at the start, on both sides of page borders and hundreds of places (many pages) back:
    every later row still depends on it, no earlier one does; seen from prompt rows, from decoded rows, and
    from the first row after a cut right behind the mark."""
    cfg, sd, path, mark, vocab = _marked_model(tmp_path, kind)
    runner = load_runner(path, torch.float32, device, max_tokens=640, max_seqs=2)
    rng = np.random.default_rng(0)
    n = 300
    for place in (0, 15, 16, 31, 32, 143, n - 2):
        toks = [int(t) for t in rng.integers(8, vocab, n)]
        toks[place] = mark
        want = lu.oracle_logits(cfg, sd, toks)
        plain = lu.oracle_logits(cfg, sd, [t if t != mark else 9 for t in toks])
        seen = np.array([lu.rel_err(plain[i:i + 1], want[i:i + 1]) for i in range(n)])      # (per row, relative to the row's spread)
        assert seen[:place].max(initial=0.0) == 0.0
        assert seen[place + 1:].min() > 100 * TOL, "the marked token does not stand out"
        assert lu.rel_err(run_cut(runner, "p", toks, [n])[-60:], want[-60:]) < TOL, place
        cuts = [place + 1] + ([n - 30 - place - 1] if n - 30 - place - 1 > 0 else [])
        tail = min(60, n - place - 1)
        assert lu.rel_err(run_cut(runner, "d", toks, cuts)[-tail:], want[-tail:]) < TOL, place
    runner.close()


# ----------------------------------------------------- command line, configuration, graphs, trace replay
def test_command_line_serves_the_model(tmp_path):
    from flexible_llm_sharding_amd import api
    from flexible_llm_sharding_amd.utils.tokenizer import write_synthetic_tokenizer
    cfg = lu.config(STACK, vocab=64, loop=LOOP)
    sd = lu.random_weights(cfg, 16)
    path = lu.write_model(str(tmp_path / "cli"), cfg, sd)
    write_synthetic_tokenizer(path, 64)
    prompts = [("w1 w2 w3", ("w4", "w5 w6")), ("w7", ("w8 w9 w10",))]
    pk = str(tmp_path / "p.pkl")
    with open(pk, "wb") as f:
        pickle.dump(prompts, f)
    out = str(tmp_path / "o.pkl")
    api.main(["--model_path", path, "--prompt_pickle", pk, "--output_file", out, "--num_gen_token", "3",
              "--num_gpus", "0" if not gpu_available() else "1", "--dtype", "float32", "--layer_num_per_shard", "2"])
    with open(out, "rb") as f:
        scores = pickle.load(f)
    assert [s.shape for s in scores] == [(2, 3, 64), (1, 3, 64)]
    assert all(abs(float(s[i, j].astype(np.float32).sum()) - 1) < 2e-2 for s in scores for i in range(s.shape[0]) for j in range(3))


def test_config_is_read_not_assumed(tmp_path):
    """The registry picks the family by config.json's architecture; every pass of a looped layer has a state
    of its own and shares its layer's weight image; every tensor of the checkpoint lands, none is invented;
    a checkpoint that contradicts the config is refused at load."""
    from flexible_llm_sharding_amd.config import LopilixConfig, load_config
    from flexible_llm_sharding_amd.models import hybrid_family, lopilix
    from flexible_llm_sharding_amd.runtime.weights import CheckpointSource, HostStore
    cfg = lu.config(STACK, loop=LOOP)
    sd = lu.random_weights(cfg, 18)
    path = lu.write_model(str(tmp_path / "c"), cfg, sd)
    c = load_config(path)
    assert isinstance(c, LopilixConfig) and hybrid_family(c) is lopilix
    assert c.layer_names() == ["embed", "l0", "l1", "l2", "l3", "l1@1", "l2@1", "l3@1", "l4", "final.norm", "head"]
    assert c.streams == 4 and c.state_width == 4 * 36 and c.residual_mult == 0.7 and c.logit_scale == 0.6 and c.hyper and c.gated
    spec = lopilix.state_spec(c)
    assert spec["paged"] == {"l0": {"k": 2 * 2 * 10, "v": 2 * 14}, "l2": {"ckr": 19}, "l2@1": {"ckr": 19}, "l4": {"k": 2 * 3 * 8, "v": 3 * 5}}
    assert spec["slots"] == {"l1": {"state": (3, 7, 9)}, "l3": {"state": (2, 20, 6)}, "l1@1": {"state": (3, 7, 9)}, "l3@1": {"state": (2, 20, 6)}}
    names = {pl.hf_name for n in c.layer_names() for pl in lopilix.placements(c, n)}
    assert names == set(sd)
    store = HostStore.from_source(CheckpointSource(c, path, torch.float32), pinned=False)
    assert store.host_buffer("l2@1") is store.host_buffer("l2") and store.host_buffer("l3") is not store.host_buffer("l2")
    for edit in (lambda d: d["layers"][0].update(type="hyena"),
                 lambda d: d["layers"][0]["mixer"].update(kv_heads=4),
                 lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7),
                 lambda d: d["layers"][2]["mixer"]["rot"].update(dims=10),
                 lambda d: d["layers"][1]["mlp"]["router"].update(top=9),
                 lambda d: d["layers"][1]["mlp"]["router"]["groups"].update(count=4),
                 lambda d: d["layers"][1]["mlp"]["router"]["groups"].update(keep=0),
                 lambda d: d.update(loop={"start": 2, "stop": 9, "times": 2}),
                 lambda d: d.update(streams=0)):
        bad = json.loads(json.dumps(cfg))
        edit(bad)
        with pytest.raises((NotImplementedError, ValueError)):
            LopilixConfig.from_dict(bad)
    wrong = json.loads(json.dumps(cfg))
    wrong["layers"][0]["mixer"]["vdim"] = 15
    lu.write_model(str(tmp_path / "w"), wrong, sd)
    with pytest.raises(ValueError):
        load_runner(str(tmp_path / "w"), torch.float32, "cpu")


@pytest.mark.gpu
def test_captured_decode_steps_equal_eager(tmp_path, monkeypatch):
    """Decode steps replay as captured HIP graphs; every replay is checked against the same steps run
    eagerly, with eager prompt steps of other requests and batch-size changes between the replays."""
    if not gpu_available():
        pytest.skip("no GPU")

    def run(graphs: bool):
        monkeypatch.setenv("FLS_DECODE_GRAPHS", "1" if graphs else "0")
        cfg, sd, runner, _ = build(tmp_path, STACK, seed=21, device="cuda:0", dtype=torch.bfloat16, max_tokens=256, max_seqs=4, loop=LOOP)
        a, b, c = (lu.tokens(n, cfg["vocab"], 60 + n) for n in (40, 33, 25))
        outs = []
        runner.step([StepEntry("a", a[:10], [9]), StepEntry("b", b[:12], [11])])
        for t in range(20):
            live = [("a", a[10 + t]), ("b", b[12 + t])] + ([("c", c[9 + t - 8])] if t >= 8 else [])
            r = runner.step([StepEntry(i, [tok], [0]) for i, tok in live])
            outs += [x[0] for x in r]
            if t == 7:
                outs.append(runner.step([StepEntry("c", c[:9], [8])])[0][0])
            if t % 5 == 0:
                torch.cuda.synchronize()
        replays = runner._decode_graphs.replays if runner._decode_graphs is not None else 0
        runner.close()
        return np.concatenate(outs, 0), replays

    eager, n0 = run(False)
    graphed, n1 = run(True)
    assert n0 == 0 and n1 >= 12
    assert np.array_equal(eager, graphed)


def test_trace_run_program_replays_steps(tmp_path):
    """bin/trace_run as a process on a two-request schedule: prompts of unequal length in one step,
    then one token each; a flushed 'done <step>' after each step, logits files for the steps that
    want some, exit code 0 at end of input."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    cfg = lu.config(STACK[:4], vocab=37, loop=(1, 3, 2))
    sd = lu.random_weights(cfg, 19)
    path = lu.write_model(str(tmp_path / "t"), cfg, sd)
    out = tmp_path / "logits"
    a, b = lu.tokens(9, 37, 4), lu.tokens(3, 37, 5)
    p = subprocess.Popen([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                          "--out", str(out), "--max-tokens", "32", "--device", "cpu"], stdin=subprocess.PIPE,
                         stdout=subprocess.PIPE, text=True, cwd=root)
    steps = [{"step": 0, "entries": [{"id": "q", "tokens": a[:7], "want": [0, 6]}, {"id": "s", "tokens": b[:1], "want": [0]}], "end": []},
             {"step": 1, "entries": [{"id": "q", "tokens": a[7:8], "want": []}, {"id": "s", "tokens": b[1:2], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "q", "tokens": a[8:], "want": [0]}, {"id": "s", "tokens": b[2:], "want": [0]}], "end": ["q", "s"]}]
    for st in steps:
        p.stdin.write(json.dumps(st) + "\n")
        p.stdin.flush()
        while True:
            line = p.stdout.readline()
            assert line, "trace_run ended early"
            if line.strip() == f"done {st['step']}":
                break
    p.stdin.close()
    assert p.wait(timeout=60) == 0
    wa, wb = lu.oracle_logits(cfg, sd, a), lu.oracle_logits(cfg, sd, b)
    got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(3, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)])
    assert not (out / "1.f32").exists()
    assert lu.rel_err(got, np.concatenate([wa[[0, 6]], wb[[0]], wa[[8]], wb[[2]]])) < TOL


def test_bench_model_builder_runs_on_cpu():
    """The benchmark's synthetic stack (bench.py --hybrid --hybrid-family lopilix) at a toy size: random layer
    images straight into a host store, a prompt step and a decode step through the runner."""
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.utils.hybrid_bench import lopilix_config, synthetic_hybrid_store
    z = dict(width=64, heads=4, kv=2, dim=16, ff=96, experts=4, top=2, eff=16, blocks=2, mh=2, mp=8, state=8, chunk=12, vocab=50)
    cfg = lopilix_config(z, times=2, streams=2)
    assert len(cfg.layer_names()) == 9
    src = synthetic_hybrid_store(cfg, "cpu", torch.float32)
    r = ShardedRunner(cfg, src, device="cpu", layer_num_per_shard=2, storage_location="cpu", compute_dtype=torch.float32,
                      state_tokens=64, state_seqs=2)
    out = r.step([StepEntry("a", list(range(20)), [19]), StepEntry("b", [1, 2, 3], [2])])
    assert out[0][0].shape == (1, 50) and np.isfinite(out[0][0]).all() and np.isfinite(out[1][0]).all()
    out = r.step([StepEntry("a", [5], [0]), StepEntry("b", [6], [])], ["a", "b"])
    assert out[1] is None and np.isfinite(out[0][0]).all() and not r.seq_cache.requests
    r.close()
