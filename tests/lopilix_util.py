"""Small random Lopilix models for the tests: configurations, weights on disk, and the oracle's
answers.  Sizes are deliberately odd and unlike each other (3 query heads per key head, head sizes
that are no powers of two, keys and values of different sizes, a rotation over part of a head, a
latent narrower than the heads it feeds, expert groups of unequal worth) and differ from layer to layer."""
import json
import os

import numpy as np
import torch

import lopilix_oracle as oracle
from flexible_llm_sharding_amd.utils.safetensors_io import save_file

SCALING = {"factor": 3.0, "original": 24, "fast": 4.0, "slow": 0.5}


def attn(heads=6, kv_heads=2, dim=10, vdim=14, rot_dims=6, base=50.0, scale=0.4, diff=0.25, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "diff": diff}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling is not None:
            m["rot"]["scaling"] = dict(scaling)
    return ("attention", m)


def hgrn(heads=3, dim=7, vdim=9):
    return ("hgrn2", {"heads": heads, "dim": dim, "vdim": vdim})


def latent(heads=3, dim=6, rot_dim=8, vdim=5, kv_rank=11, base=100.0, scaling=SCALING, scale=0.3):
    rot = {"dims": rot_dim, "base": base}
    if scaling is not None:
        rot["scaling"] = dict(scaling)
    return ("latent_attention", {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot,
                                 "scale": scale})


def dense(ff=20):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=12, groups=(3, 2), scale=1.7):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "router": r, "expert": {"ff": ff}}


def config(layers, width=36, vocab=53, eps=1e-5, mult=0.7, streams=4, logit_scale=0.6, loop=None, max_positions=400):
    """layers: [((type, mixer dict), mlp dict or None)] -> config.json's content."""
    d = {"architecture": "Lopilix", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult,
         "streams": streams, "logit_scale": logit_scale, "max_positions": max_positions,
         "layers": [{"type": t, "mixer": json.loads(json.dumps(m)), "mlp": json.loads(json.dumps(f))} for (t, m), f in layers]}
    if loop:
        d["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return d


def random_weights(cfg, seed=0, std=0.3):
    g = torch.Generator().manual_seed(seed)
    D, S = cfg["width"], cfg["streams"]

    def mat(*shape, s=std):
        return torch.randn(*shape, generator=g) * s

    sd = {"embed": mat(cfg["vocab"], D, s=1.0), "pos": mat(cfg["max_positions"], D, s=0.5), "final.norm": 1.0 + mat(D, s=0.3)}
    for i, l in enumerate(cfg["layers"]):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        for q in (1, 2):
            if q == 2 and l["mlp"] is None:
                break
            sd[f"{p}norm{q}"] = 1.0 + mat(D, s=0.3)
            sd[f"{p}hc{q}.in"] = 1.0 / S + mat(S, s=0.3)
            sd[f"{p}hc{q}.out"] = 1.0 + mat(S, s=0.4)
            sd[f"{p}hc{q}.mix"] = torch.eye(S) + mat(S, S, s=0.25)
            sd[f"{p}rg{q}"] = mat(D, D, s=0.2)
            sd[f"{p}rg{q}.b"] = mat(D, s=0.5)
        if l["type"] == "attention":
            H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            sd.update({x + "q": mat(2 * H * d, D), x + "k": mat(2 * G * d, D), x + "v": mat(G * dv, D), x + "o": mat(D, H * dv),
                       x + "q.norm": 1.0 + mat(d, s=0.3), x + "k.norm": 1.0 + mat(d, s=0.3)})
            for n in ("lq1", "lk1", "lq2", "lk2"):
                sd[x + n] = mat(d, s=0.3)
        elif l["type"] == "hgrn2":
            H, d, dv = m["heads"], m["dim"], m["vdim"]
            sd.update({x + "q": mat(H * d, D), x + "f": mat(H * d, D), x + "f.b": mat(H * d, s=1.0), x + "v": mat(H * dv, D),
                       x + "lower": 0.9 * torch.rand(H * d, generator=g), x + "norm": 1.0 + mat(dv, s=0.3), x + "o": mat(D, H * dv)})
        else:
            H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            sd.update({x + "q": mat(H * (d + dr), D), x + "dkv": mat(r + dr, D), x + "dkv.norm": 1.0 + mat(r, s=0.3),
                       x + "uk": mat(H * d, r), x + "uv": mat(H * dv, r), x + "g": mat(H * dv, D), x + "o": mat(D, H * dv)})
        f = l["mlp"]
        if f is None:
            continue
        y = p + "mlp."
        if f["kind"] == "dense":
            ff = f["ff"]
            sd.update({y + "gate": mat(ff, D), y + "gate.b": mat(ff), y + "up": mat(ff, D), y + "up.b": mat(ff),
                       y + "down": mat(D, ff), y + "down.b": mat(D)})
        else:
            sd[y + "router"] = mat(f["router"]["experts"], D, s=0.8)
            for e in range(f["router"]["experts"]):
                sd.update({f"{y}e{e}.up": mat(f["expert"]["ff"], D), f"{y}e{e}.down": mat(D, f["expert"]["ff"])})
    return {k: v.to(torch.bfloat16) for k, v in sd.items()}


def write_model(path, cfg, sd):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(sd, os.path.join(path, "model.safetensors"))
    return path


def f64(sd):
    return {k: v.to(torch.float64) for k, v in sd.items()}


def oracle_logits(cfg, sd, tokens, trace=None):
    return oracle.forward(f64(sd), cfg, list(tokens), trace).numpy()


def row_errs(got, want):
    """Per row: mean-free RMS difference of the logits over the RMS of the wanted row."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / (np.sqrt((w ** 2).mean(-1)) + 1e-12)


def rel_err(got, want):
    """The worst row of ``row_errs``."""
    return float(row_errs(got, want).max())


def tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()
