"""Small random Gizezen models for the tests: configurations, weights on disk, and the oracle's
answers.  Sizes are deliberately odd and unlike each other (3 query heads per key head, head sizes
that are no powers of two, keys and values of different sizes, windows that are no multiples of the
page size, a rotation over part of a head with all three frequency bands of the rescaling, tap
counts from 1 to 5) and differ from layer to layer."""
import json
import os

import numpy as np
import torch

import gizezen_oracle as oracle
from flexible_llm_sharding_amd.utils.safetensors_io import save_file

SCALING = {"factor": 4.0, "low": 2.0, "high": 6.0, "original": 96}


def attn(heads=6, kv_heads=2, dim=10, vdim=14, size=9, rot_dims=6, base=50.0, scaling=SCALING, conv=3, scale=0.4, kv_from=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "mask": {"size": size},
         "rot": {"dims": rot_dims, "base": base}, "scale": scale}
    if scaling is not None:
        m["rot"]["scaling"] = dict(scaling)
    if kv_from is not None:
        m["kv_from"] = kv_from
    return m


def moe(experts=5, top=2, ff=12, shared=20):
    m = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def config(layers, width=36, vocab=53, eps=1e-5, mult=0.8, emb=1.7):
    """layers: [(mixer dict, mlp dict or None)] -> config.json's content."""
    return {"architecture": "Gizezen", "width": width, "vocab": vocab, "norm": {"eps": eps}, "residual_mult": mult,
            "embedding": {"scale": emb},
            "layers": [{"type": "attention", "mixer": json.loads(json.dumps(m)), "mlp": json.loads(json.dumps(f))} for m, f in layers]}


def random_weights(cfg, seed=0, std=0.3):
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def mat(*shape, s=std):
        return torch.randn(*shape, generator=g) * s

    def norm(name):
        return {name: 1.0 + mat(D, s=0.3), name + ".b": mat(D, s=0.2), name + ".alpha": torch.tensor(0.5) + 0.3 * torch.rand((), generator=g)}

    sd = {"embed": mat(cfg["vocab"], D, s=1.0), "head": mat(cfg["vocab"], D), **norm("final.norm")}
    for i, l in enumerate(cfg["layers"]):
        p, m, x = f"l{i}.", l["mixer"], f"l{i}.mix."
        H, G, d, dv, taps = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
        sd.update(norm(p + "norm1"))
        sd.update({x + "q": mat(H * d, D), x + "q.conv": mat(H * d, taps, s=0.6), x + "g": mat(H, D, s=0.6), x + "o": mat(D, H * dv)})
        if m.get("kv_from") is None:
            sd.update({x + "k": mat(G * d, D), x + "k.conv": mat(G * d, taps, s=0.6),
                       x + "v": mat(G * dv, D), x + "v.conv": mat(G * dv, taps, s=0.6)})
        f = l["mlp"]
        if f is not None:
            y = p + "mlp."
            sd.update(norm(p + "norm2"))
            sd[y + "router"] = mat(f["router"]["experts"], D, s=0.8)
            for e in range(f["router"]["experts"]):
                sd.update({f"{y}e{e}.gate": mat(f["expert"]["ff"], D), f"{y}e{e}.up": mat(f["expert"]["ff"], D),
                           f"{y}e{e}.down": mat(D, f["expert"]["ff"])})
            if f.get("shared"):
                fs = f["shared"]["ff"]
                sd.update({y + "shared.gate": mat(fs, D), y + "shared.up": mat(fs, D), y + "shared.down": mat(D, fs),
                           y + "shared.sg": mat(1, D, s=0.6)})
    return {k: v.to(torch.bfloat16) for k, v in sd.items()}


def write_model(path, cfg, sd):
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file(sd, os.path.join(path, "model.safetensors"))
    return path


def oracle_logits(cfg, sd, tokens):
    return oracle.forward(cfg, sd, list(tokens)).numpy()


def rel_err(got, want):
    """Mean-free RMS difference of logit rows over the RMS of the wanted rows (the worst row)."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return float((np.sqrt((d ** 2).mean(-1)) / (np.sqrt((w ** 2).mean(-1)) + 1e-12)).max())


def tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()
