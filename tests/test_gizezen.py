"""Gizezen through the framework (config registry, weight images, sequence state cache, step
scheduler, kernels) against the plain float64 oracle in ``gizezen_oracle.py``.

Every test runs on the CPU backend (plain PyTorch ops) and, marked ``gpu``, on the HIP kernels.  The
models are tiny and random; fp32 matrix products make the comparison sharp (a window one token off,
a lost convolution history, a forgotten silent softmax entry or a wrong page shows as an error
thousands of times the tolerance), and two tests run the bf16 mode.  Where random weights would hide
a fault, the weights are set so that one key dominates."""
import json
import math
import os
import pickle
import subprocess
import sys

import numpy as np
import pytest
import torch

import gizezen_oracle as oracle
import gizezen_util as gu
from conftest import gpu_available
from flexible_llm_sharding_amd.runtime.batch import StepEntry
from flexible_llm_sharding_amd.serve import generate, load_runner

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
TOL = 2e-4          # fp32 products against float64, relative to a logit row's spread


@pytest.fixture(autouse=True)
def _need_gpu(request):
    params = getattr(getattr(request.node, "callspec", None), "params", {})
    if "cuda" in str(params.get("device", "")) and not gpu_available():
        pytest.skip("no GPU")


def build(tmp_path, layers, seed=0, dtype=torch.float32, device="cpu", **kw):
    cfg = gu.config(layers, **{k: v for k, v in kw.items() if k in ("width", "vocab", "eps", "mult", "emb")})
    sd = gu.random_weights(cfg, seed, **({"std": kw["std"]} if "std" in kw else {}))
    path = gu.write_model(str(tmp_path / f"m{seed}"), cfg, sd)
    runner = load_runner(path, dtype, device, max_tokens=kw.get("max_tokens", 64), max_seqs=kw.get("max_seqs", 2),
                         layer_num_per_shard=kw.get("lnps"), token_budget=kw.get("token_budget", 16384))
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


# keys of its own; a reader of layer 0 with another window and more query heads; a second owner without a feed-forward
# (multi-head, whole head rotated, unscaled frequencies, four taps); two readers of layer 2, one without a shared expert
STACK = [(gu.attn(), gu.moe()),
         (gu.attn(heads=4, size=13, conv=2, scale=0.7, kv_from=0), gu.moe(experts=3, top=1, ff=9, shared=7)),
         (gu.attn(heads=3, kv_heads=3, dim=8, vdim=5, size=5, rot_dims=8, base=1000.0, scaling=None, conv=4), None),
         (gu.attn(heads=3, kv_heads=3, dim=8, vdim=5, size=21, rot_dims=8, base=1000.0, scaling=None, conv=1, kv_from=2),
          gu.moe(experts=4, top=4, ff=10, shared=0)),
         (gu.attn(heads=6, kv_heads=3, dim=8, vdim=5, size=3, rot_dims=8, base=1000.0, scaling=None, conv=5, kv_from=2), gu.moe())]


# ------------------------------------------------------------------ each mechanism alone
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name,layers,kw", [
    ("attention", [(gu.attn(scale=1.5), None)], {}),
    ("one-head-window-1", [(gu.attn(heads=1, kv_heads=1, dim=4, vdim=3, size=1, rot_dims=2), None)], {}),
    ("multi-head-full-rotation-unscaled", [(gu.attn(heads=3, kv_heads=3, dim=8, vdim=8, rot_dims=8, scaling=None), None)], {}),
    ("shared-keys", [(gu.attn(), None), (gu.attn(size=4, conv=2, kv_from=0), None)], {}),
    ("no-conv-taps", [(gu.attn(conv=1), gu.moe())], {}),
    ("seven-taps", [(gu.attn(conv=7), None)], {}),
    ("ten-taps", [(gu.attn(conv=10), None)], {}),
    ("unit-multipliers", [(gu.attn(), gu.moe())], {"mult": 1.0, "emb": 1.0}),
    ("experts-top-1", [(gu.attn(size=2), gu.moe(experts=7, top=1, shared=0))], {}),
    ("experts-all-chosen-with-shared", [(gu.attn(size=2), gu.moe(experts=3, top=3, ff=30, shared=50))], {}),
    ("width-not-a-multiple-of-four", [(gu.attn(), gu.moe())], {"width": 34}),
])
def test_mechanism_alone(tmp_path, device, name, layers, kw):
    cfg, sd, runner, _ = build(tmp_path, layers, seed=3, device=device, **kw)
    toks = gu.tokens(45, cfg["vocab"], 1)
    want = gu.oracle_logits(cfg, sd, toks)
    assert gu.rel_err(run_cut(runner, "a", toks, [len(toks)]), want) < TOL
    assert gu.rel_err(run_cut(runner, "b", toks, [30, 2]), want) < TOL
    runner.close()


def test_oracle_parts_agree_with_their_definitions():
    """The oracle's own pieces on hand-made inputs: the window, the tap order of the convolution, the
    rotation of a pair, the three bands of the frequency rescaling, the silent softmax entry, routing."""
    assert [j for j in range(12) if oracle.sees(10, j, 3)] == [8, 9, 10] and not oracle.sees(3, 4, 9)
    u = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    w = torch.tensor([[0.5, 0.25, 2.0]], dtype=torch.float64)          # taps 3: w[:, 2] weighs the current row
    assert torch.allclose(oracle.short_conv(u, w)[:, 0], torch.tensor([2.0, 20 + 0.25, 200 + 2.5 + 0.5], dtype=torch.float64))
    x = torch.tensor([[[0.0, 0.0, 5.0, 6.0]], [[1.0, 0.0, 5.0, 6.0]]], dtype=torch.float64)
    r = oracle.rotate(x, {"dims": 2, "base": 100.0})
    assert torch.allclose(r[1, 0], torch.tensor([math.cos(1.0), math.sin(1.0), 5.0, 6.0], dtype=torch.float64))
    rot = {"dims": 16, "base": 100.0, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}}
    f, f0 = oracle.rot_freqs(rot), oracle.rot_freqs({"dims": 16, "base": 100.0})
    ratio = [a / b for a, b in zip(f, f0)]
    assert ratio[0] == 1.0 and abs(ratio[-1] - 1 / 8) < 1e-12 and any(1 / 8 + 1e-3 < r < 1 - 1e-3 for r in ratio)
    i = next(k for k, r in enumerate(ratio) if 1 / 8 + 1e-3 < r < 1 - 1e-3)        # a blended one, worked out by hand
    s = (64 * f0[i] / (2 * math.pi) - 1.0) / 3.0
    assert abs(f[i] - ((1 - s) * f0[i] / 8 + s * f0[i])) < 1e-15
    p = oracle.sink_softmax(torch.tensor([0.0, math.log(2.0)], dtype=torch.float64))
    assert torch.allclose(p, torch.tensor([0.25, 0.5], dtype=torch.float64))
    assert oracle.sink_softmax(torch.tensor([-50.0, -60.0], dtype=torch.float64)).sum() < 1e-20
    ids, wts = oracle.route(torch.tensor([[0.0, 3.0, 1.0, 3.0 - math.log(3.0)]], dtype=torch.float64), 2)
    assert ids.tolist() == [[1, 3]] and torch.allclose(wts, torch.tensor([[0.75, 0.25]], dtype=torch.float64))


# ----------------------------------------------- prompts, portions, decoding, first tokens
@pytest.mark.parametrize("device", DEVICES)
def test_prefill_portions_and_decode(tmp_path, device):
    """The same sequence whole, token by token, and in portions of 2, 3, 7, 16 and 17 tokens: windows,
    shared keys and the convolutions' histories all cross the cuts."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=5, device=device)
    toks = gu.tokens(50, cfg["vocab"], 2)
    want = gu.oracle_logits(cfg, sd, toks)
    for cuts in ([50], [], [2, 2, 3, 7, 16, 17], [17, 16, 2], [1, 2, 40]):
        assert gu.rel_err(run_cut(runner, "r", toks, cuts), want) < TOL, cuts
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_over_windows_and_pages(tmp_path, device):
    """A short prompt, then 120 decoded tokens: every window passes over decoded tokens, pages of 16
    fill, and the pages behind the widest window go back to the pool while the request lives."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=6, device=device)
    toks = gu.tokens(125, cfg["vocab"], 7)
    got = run_cut(runner, "r", toks, [5], end=False)
    assert gu.rel_err(got, gu.oracle_logits(cfg, sd, toks)) < TOL
    cache = runner.seq_cache
    req = cache.requests["r"]
    assert cache.pages_trimmed > 0 and req.pages[0] < 0 and req.pages[-1] >= 0
    cache.release("r")
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(tmp_path, device):
    """Sequences of one, two and three tokens (shorter than the convolutions and the windows), whole and decoded."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=8, device=device)
    for n in (1, 2, 3):
        toks = gu.tokens(n, cfg["vocab"], 20 + n)
        want = gu.oracle_logits(cfg, sd, toks)
        assert gu.rel_err(run_cut(runner, "w", toks, [n]), want) < TOL
        assert gu.rel_err(run_cut(runner, "d", toks, []), want) < TOL
    runner.close()


# ------------------------------------------------------------ batches, pages and slots
@pytest.mark.parametrize("device", DEVICES)
def test_unequal_batch_equals_each_alone(tmp_path, device):
    """Requests of 1, 9, 33 and 50 tokens in one step, then decoded together while the short ones
    finish first; also cut into two micro-batches by a small token budget."""
    for budget in (16384, 40):
        cfg, sd, runner, _ = build(tmp_path, STACK, seed=9, device=device, token_budget=budget)
        lens, extra = [1, 9, 33, 50], [3, 12, 0, 6]
        seqs = [gu.tokens(n + e, cfg["vocab"], 30 + i) for i, (n, e) in enumerate(zip(lens, extra))]
        want = [gu.oracle_logits(cfg, sd, s) for s in seqs]
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
            assert gu.rel_err(np.concatenate(got[i], 0), want[i]) < TOL, (budget, i)
        assert not runner.seq_cache.requests
        runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_pages_and_slots_used_again(tmp_path, device):
    """Requests come and go through pools of two slots and a few pages: whoever inherits a page or a
    slot (with the last owner's keys, values and convolution histories still in it) computes what it
    computes alone, and pools that run out grow without disturbing the live request."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=11, device=device, max_tokens=40, max_seqs=2)
    cache = runner.seq_cache
    a, b, c = (gu.tokens(n, cfg["vocab"], 40 + n) for n in (37, 22, 41))
    wa, wb, wc = (gu.oracle_logits(cfg, sd, s) for s in (a, b, c))
    assert gu.rel_err(run_cut(runner, "a", a, [30]), wa) < TOL
    ga = run_cut(runner, "a2", a, [10, 2], end=False)                       # stays alive
    gb = run_cut(runner, "b", b, [22])                                      # inherits a's first slot
    assert cache.slots_reused > 0 and cache.pages_reused > 0
    gc = run_cut(runner, "c", c, [3, 30])
    n0 = cache.n_slots
    others = [run_cut(runner, f"x{i}", b, [5], end=False) for i in range(3)]    # more requests than slots
    assert cache.n_slots > n0
    tail = runner.step([StepEntry("a2", [a[0]], [0])], ["a2"])[0][0]         # a2's state survived the growth
    assert gu.rel_err(tail, gu.oracle_logits(cfg, sd, a + [a[0]])[-1:]) < TOL
    for g, w in ((ga, wa), (gb, wb), (gc, wc)) + tuple((o, wb) for o in others):
        assert gu.rel_err(g, w) < TOL
    runner.close()


# ------------------------------------------- one key that stands out, at every kind of edge
def _marked_model(tmp_path, size, reader_size=None):
    """One attention layer without convolution whose weights make the marked token's key the only one that
    any query likes: the norm's bias gives every token the same query direction u and every other token the
    key -u; the marked token's embedding flips its key to +u and makes its value large.  Scores are then
    about +scale * dim for the marked key and -scale * dim for all others, so that next to the silent entry
    of score 0 a row's output is about the marked value if it sees the marked key and about zero if not.
    ``reader_size``: a second layer that reads the first one's keys and values through a window of its own."""
    D, vocab, mark, d = 24, 40, 7, 8
    layers = [(gu.attn(heads=2, kv_heads=1, dim=d, vdim=6, size=size, rot_dims=2, base=1e6, scaling=None, conv=1, scale=1.6), None)]
    if reader_size:
        layers.append((gu.attn(heads=2, kv_heads=1, dim=d, vdim=6, size=reader_size, rot_dims=2, base=1e6, scaling=None, conv=1,
                               scale=1.6, kv_from=0), None))
    cfg = gu.config(layers, width=D, vocab=vocab, mult=1.0, emb=1.0)
    sd = {k: v.float() for k, v in gu.random_weights(cfg, 12, std=0.05).items()}
    u = torch.tensor([0.0, 0.0, 1.0, -1.0, 1.0, 1.0, -1.0, 1.0])            # (entries 0, 1 are the rotated pair: left out)
    sd["embed"][:, :2] = 0.0
    sd["embed"][mark, 1] = 8.0                                             # tanh saturates: channel 1 reads +1 for the mark
    for i in range(len(layers)):
        p = f"l{i}."
        sd[p + "norm1"][:2] = torch.tensor([0.0, 2.0])                     # channel 0: the constant 1; channel 1: -1, or +1 for the mark
        sd[p + "norm1.b"][:2] = torch.tensor([1.0, -1.0])
        sd[p + "norm1.alpha"] = torch.tensor(1.0)
        sd[p + "mix.q"] *= 0.2
        sd[p + "mix.q"][:, 0] = torch.cat([u, u])
        sd[p + "mix.q.conv"][:] = 1.0
        sd[p + "mix.g"][:, 0] = 2.0
    sd["l0.mix.k"] *= 0.2
    sd["l0.mix.k"][:, 1] = u
    sd["l0.mix.k.conv"][:] = 1.0
    sd["l0.mix.v.conv"][:] = 1.0
    sd["l0.mix.v"][:, 1] = 3.0
    sd = {k: v.to(torch.bfloat16) for k, v in sd.items()}
    return cfg, sd, gu.write_model(str(tmp_path / f"edge{size}_{reader_size}"), cfg, sd), mark, vocab


def _unmarked(toks, mark):
    return [t if t != mark else 9 for t in toks]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("size,reader", [(21, None), (21, 34), (34, 21)])
def test_one_key_stands_out_at_window_edges(tmp_path, device, size, reader):
    """The marked token far back, on page borders, at the window's last and first place and one place
    outside, seen from a prompt position, from a decoded one, and from the first decoded token after a
    prompt that ends where the window's edge lies; alone, and through a second layer that shares the keys
    with a narrower or a wider window of its own."""
    cfg, sd, path, mark, vocab = _marked_model(tmp_path, size, reader)
    runner = load_runner(path, torch.float32, device, max_tokens=128, max_seqs=2)
    rng = np.random.default_rng(0)
    n, widest = 70, max(size, reader or 0)
    for place in (0, 15, 16, 31, 32, n - widest - 1, n - widest, n - size, n - size + 1, n - 2):
        toks = [int(t) for t in rng.integers(8, vocab, n)]
        toks[place] = mark
        want = gu.oracle_logits(cfg, sd, toks)
        seen = np.abs(want - gu.oracle_logits(cfg, sd, _unmarked(toks, mark))).max(-1)
        inside = [i for i in range(place + 1, n) if i - place < min(size, reader or size)]
        outside = [i for i in range(place + widest, n)] if not reader else []
        assert not inside or seen[inside].min() > 50 * TOL * np.abs(want).max(), "the marked key does not stand out"
        assert not outside or seen[outside].max() == 0.0
        assert gu.rel_err(run_cut(runner, "p", toks, [n]), want) < TOL, place
        assert gu.rel_err(run_cut(runner, "d", toks, [place + 1]), want) < TOL, place
        assert gu.rel_err(run_cut(runner, "e", toks, [min(n, place + size - 1)]), want) < TOL, place
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_a_far_key_among_hundreds_and_rows_that_see_no_liked_key(tmp_path, device):
    """A window of 260 over sequences of 300: the marked key lies hundreds of places (and many pages) back
    and still decides the row, or has just left the window; rows whose window holds no liked key give
    their weight to the silent entry and come out near zero, which a softmax without it would not."""
    size = 260
    cfg, sd, path, mark, vocab = _marked_model(tmp_path, size)
    runner = load_runner(path, torch.float32, device, max_tokens=640, max_seqs=2)
    rng = np.random.default_rng(1)
    n = 300
    for place in (3, n - size - 1, n - size, n - size + 1):
        toks = [int(t) for t in rng.integers(8, vocab, n)]
        toks[place] = mark
        want = gu.oracle_logits(cfg, sd, toks)
        seen = np.abs(want - gu.oracle_logits(cfg, sd, _unmarked(toks, mark))).max(-1)
        assert (seen[n - 1] > 50 * TOL * np.abs(want).max()) == (n - 1 - place < size), place
        assert gu.rel_err(run_cut(runner, "p", toks, [n])[-45:], want[-45:]) < TOL, place
        assert gu.rel_err(run_cut(runner, "d", toks, [n - 40])[-45:], want[-45:]) < TOL, place
    # without the mark every key scores about -scale * dim: the mixer's output is about e^-12 of a value
    toks = [int(t) for t in rng.integers(8, vocab, 40)]
    layers_out = []
    oracle.forward(cfg, sd, toks, layers_out)
    x0 = sd["embed"].double()[torch.tensor(toks)]
    assert (layers_out[0] - x0).abs().max() < 1e-3 * x0.abs().max()
    assert gu.rel_err(run_cut(runner, "s", toks, [17]), gu.oracle_logits(cfg, sd, toks)) < TOL
    runner.close()


# ----------------------------------------------------- shards, bf16, generation, command line
@pytest.mark.parametrize("device", DEVICES)
def test_one_layer_per_shard_streams_weights(tmp_path, device):
    cfg = gu.config(STACK)
    sd = gu.random_weights(cfg, 13)
    path = gu.write_model(str(tmp_path / "s"), cfg, sd)
    runner = load_runner(path, torch.float32, device, max_tokens=64, layer_num_per_shard=1, resident=False)
    toks = gu.tokens(40, cfg["vocab"], 3)
    assert gu.rel_err(run_cut(runner, "r", toks, [20, 2]), gu.oracle_logits(cfg, sd, toks)) < TOL
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_bf16_products_stay_close(tmp_path, device):
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=14, device=device, dtype=torch.bfloat16)
    toks = gu.tokens(40, cfg["vocab"], 4)
    want = gu.oracle_logits(cfg, sd, toks)
    whole, cut = run_cut(runner, "a", toks, [40]), run_cut(runner, "b", toks, [9, 2])
    assert gu.rel_err(whole, want) < 0.08 and gu.rel_err(cut, want) < 0.08
    assert gu.rel_err(cut, whole) < 0.05
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_head_sizes_of_the_matrix_core_kernel(tmp_path, device):
    """bf16 with key sizes of 64 and 128 and value sizes of 128 and 64, which the matrix-core prompt
    attention serves on the GPU (silent entry and head gates in its epilogue): a prompt of several row
    tiles, a portion that continues it, then decoding past the windows.  Whole-prompt and decoded logits
    both stay within bf16 rounding of the oracle, and of each other."""
    layers = [(gu.attn(heads=4, kv_heads=2, dim=64, vdim=128, size=150, rot_dims=32, base=1e4, scale=0.12), gu.moe()),
              (gu.attn(heads=2, kv_heads=2, dim=64, vdim=128, size=33, rot_dims=32, base=1e4, scale=0.12, kv_from=0), None),
              (gu.attn(heads=2, kv_heads=1, dim=128, vdim=64, size=40, rot_dims=128, base=1e4, scaling=None, scale=0.09), None)]
    cfg, sd, runner, _ = build(tmp_path, layers, seed=23, device=device, dtype=torch.bfloat16, max_tokens=512, std=0.2)
    toks = gu.tokens(230, cfg["vocab"], 6)
    want = gu.oracle_logits(cfg, sd, toks)
    whole = run_cut(runner, "a", toks, [230])
    cut = run_cut(runner, "b", toks, [150, 40])
    assert gu.rel_err(whole, want) < 0.08 and gu.rel_err(cut, want) < 0.08
    assert gu.rel_err(cut, whole) < 0.06
    runner.close()


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_scheduler(tmp_path, device):
    """serve.generate: prompts of unequal length, 12 new tokens each; the tokens are the oracle's
    greedy continuation (recomputed from scratch at every step)."""
    cfg, sd, runner, _ = build(tmp_path, STACK, seed=15, device=device)
    prompts = [gu.tokens(n, cfg["vocab"], 50 + n) for n in (3, 17, 26)]
    got = generate(runner, prompts, 12)
    for p, g in zip(prompts, got):
        seq = list(p)
        for t in g:
            z = gu.oracle_logits(cfg, sd, seq)[-1]
            top2 = np.sort(z)[-2:]
            if top2[1] - top2[0] > 1e-3:              # (a tie within rounding may go either way)
                assert t == int(z.argmax())
            seq.append(t)
    assert not runner.seq_cache.requests
    runner.close()


def test_command_line_serves_the_model(tmp_path):
    from flexible_llm_sharding_amd import api
    from flexible_llm_sharding_amd.utils.tokenizer import write_synthetic_tokenizer
    cfg = gu.config(STACK, vocab=64)
    sd = gu.random_weights(cfg, 16)
    path = gu.write_model(str(tmp_path / "cli"), cfg, sd)
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
    """The registry picks the family by config.json's architecture; what a layer may share is checked; a
    checkpoint that contradicts the config is refused at load; absent optional parts are absent."""
    from flexible_llm_sharding_amd.config import GizezenConfig, load_config
    from flexible_llm_sharding_amd.models import gizezen, hybrid_family
    cfg = gu.config(STACK)
    sd = gu.random_weights(cfg, 18)
    path = gu.write_model(str(tmp_path / "c"), cfg, sd)
    c = load_config(path)
    assert isinstance(c, GizezenConfig) and hybrid_family(c) is gizezen
    assert c.kv_owner(1) == 0 and c.kv_owner(4) == 2 and c.residual_mult == 0.8 and c.embedding_scale == 1.7
    spec = gizezen.state_spec(c)
    assert sorted(spec["paged"]) == ["l0", "l2"] and spec["alias"] == {"l1": "l0", "l3": "l2", "l4": "l2"}
    assert spec["slots"]["l1"]["conv"] == (1, 4 * 10) and spec["slots"]["l2"]["conv"] == (3, 3 * 8 + 3 * 8 + 3 * 5)
    assert [h[1] for h in spec["horizons"]] == [9, 13, 5, 21, 3]
    names = {pl.hf_name for n in c.layer_names() for pl in gizezen.placements(c, n)}
    assert names == set(sd)                                   # every tensor of the checkpoint lands, none is invented
    for edit in (lambda d: d["layers"][0].update(type="hyena"),
                 lambda d: d["layers"][1]["mixer"].update(dim=12),
                 lambda d: d["layers"][3]["mixer"].update(kv_from=1),
                 lambda d: d["layers"][4]["mixer"].update(kv_from=4),
                 lambda d: d["layers"][0]["mixer"]["rot"].update(dims=7),
                 lambda d: d["layers"][0]["mlp"]["router"].update(top=9)):
        bad = json.loads(json.dumps(cfg))
        edit(bad)
        with pytest.raises((NotImplementedError, ValueError)):
            GizezenConfig.from_dict(bad)
    wrong = json.loads(json.dumps(cfg))
    wrong["layers"][0]["mixer"]["vdim"] = 15
    wrong["layers"][1]["mixer"]["vdim"] = 15
    gu.write_model(str(tmp_path / "w"), wrong, sd)
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
        cfg, sd, runner, _ = build(tmp_path, STACK, seed=21, device="cuda:0", dtype=torch.bfloat16, max_tokens=256, max_seqs=4)
        a, b, c = (gu.tokens(n, cfg["vocab"], 60 + n) for n in (40, 33, 25))
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
    cfg = gu.config(STACK[:4], vocab=37)
    sd = gu.random_weights(cfg, 19)
    path = gu.write_model(str(tmp_path / "t"), cfg, sd)
    out = tmp_path / "logits"
    a, b = gu.tokens(9, 37, 4), gu.tokens(3, 37, 5)
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
    wa, wb = gu.oracle_logits(cfg, sd, a), gu.oracle_logits(cfg, sd, b)
    got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(3, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(2, -1)])
    assert not (out / "1.f32").exists()
    assert gu.rel_err(got, np.concatenate([wa[[0, 6]], wb[[0]], wa[[8]], wb[[2]]])) < TOL


def test_bench_model_builder_runs_on_cpu():
    """The benchmark's synthetic stacks (bench.py --hybrid --hybrid-family gizezen) at a toy size: random layer
    images straight into a host store, a prompt step and a decode step through the runner."""
    from flexible_llm_sharding_amd.engine import ShardedRunner
    from flexible_llm_sharding_amd.utils.hybrid_bench import gizezen_config, kagolix_attention_moe_config, synthetic_hybrid_store
    z = dict(width=64, heads=4, kv=2, dim=16, ff=96, experts=4, top=2, eff=16, blocks=2, mh=2, mp=8, state=8, chunk=12, vocab=50)
    for cfg in (gizezen_config(z, repeats=1), kagolix_attention_moe_config(z, 2)):
        src = synthetic_hybrid_store(cfg, "cpu", torch.float32)
        r = ShardedRunner(cfg, src, device="cpu", layer_num_per_shard=2, storage_location="cpu", compute_dtype=torch.float32,
                          state_tokens=64, state_seqs=2)
        out = r.step([StepEntry("a", list(range(20)), [19]), StepEntry("b", [1, 2, 3], [2])])
        assert out[0][0].shape == (1, 50) and np.isfinite(out[0][0]).all() and np.isfinite(out[1][0]).all()
        out = r.step([StepEntry("a", [5], [0]), StepEntry("b", [6], [])], ["a", "b"])
        assert out[1] is None and np.isfinite(out[0][0]).all() and not r.seq_cache.requests
        r.close()
