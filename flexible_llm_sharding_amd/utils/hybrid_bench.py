"""Throughput of a hybrid stack next to the closest existing model at equal size: ``bench.py --hybrid``
(Kagolix beside a Mixtral-structured stack; ``--hybrid-family sisavik``: Sisavik beside Kagolix;
``--hybrid-family gizezen``: Gizezen beside a Kagolix stack of attention layers with experts;
``--hybrid-family lopilix``: Lopilix beside the Kagolix stack of attention, recurrent and state-space layers).

Random weights at sizes that resemble a real model's layers.  Three parts, one JSON line each:

* ``hybrid``: prefill (B prompts of L tokens in one step) and decode (B requests at context L, one
  token each per step) through ``ShardedRunner.step`` with resident weights;
* ``dense``: the closest existing model, a Mixtral-structured stack of the same width, heads, ff,
  experts and depth, through the scoring engine: a full pass over B prompts of L tokens (prefill) and
  generation steps on the prefix / suffix K/V caches (decode);
* ``kernels``: each hybrid kernel alone at the prefill and decode shapes, with its rate against the
  chip's dense bf16 matrix peak or HBM bandwidth, and the dense family's GEMM and RMSNorm likewise.
"""
from __future__ import annotations

import json
import time
from typing import Dict, List

import numpy as np
import torch

from ..config import GizezenConfig, KagolixConfig, LopilixConfig, ModelConfig, SisavikConfig

PEAK_FLOPS = 2.5e15        # dense bf16 / fp16 matrix peak of one MI355X
PEAK_BYTES = 8.0e12        # HBM3E

SIZES = {
    # width, heads, kv, dim, ff, experts, top, expert ff, rglru blocks, mamba heads x vdim, state, chunk
    "s": dict(width=2048, heads=16, kv=4, dim=128, ff=8192, experts=8, top=2, eff=2048, blocks=16, mh=32, mp=64,
              state=128, chunk=1024, vocab=32000),
    "m": dict(width=4096, heads=32, kv=8, dim=128, ff=14336, experts=8, top=2, eff=4096, blocks=16, mh=64, mp=64,
              state=128, chunk=2048, vocab=32000),
}


def hybrid_config(z: dict, repeats: int = 2) -> KagolixConfig:
    att = {"type": "attention", "mixer": {"heads": z["heads"], "kv_heads": z["kv"], "dim": z["dim"], "vdim": z["dim"],
                                           "mask": {"size": z["chunk"]}, "scale": z["dim"] ** -0.5, "softcap": 30.0}}
    rg = {"type": "rglru", "mixer": {"width": z["width"], "blocks": z["blocks"], "conv": 4}}
    mb = {"type": "mamba2", "mixer": {"heads": z["mh"], "vdim": z["mp"], "state": z["state"], "groups": 1,
                                      "norm_groups": 1, "conv": 4}}
    dense = {"kind": "dense", "ff": z["ff"]}
    moe = {"kind": "moe", "expert": {"ff": z["eff"]}, "router": {"experts": z["experts"], "top": z["top"]}}
    layers = []
    for _ in range(repeats):
        layers += [dict(att, mlp=dense), dict(rg, mlp=moe), dict(mb, mlp=moe)]
    return KagolixConfig.from_dict({"architecture": "Kagolix", "width": z["width"], "vocab": z["vocab"],
                                    "norm": {"eps": 1e-6, "groups": 2}, "logit_softcap": 30.0, "layers": layers})


def sisavik_config(z: dict, repeats: int = 2) -> SisavikConfig:
    """Latent attention, a parallel pair, and a latent attention that reads the first one's latent, each
    with a dense feed-forward: per-head sizes, ranks and windows of the order real models use."""
    d = z["dim"]
    lat = {"heads": z["heads"], "dim": d // 2, "rot_dim": d // 2, "vdim": d, "kv_rank": 4 * d, "q_rank": 3 * z["width"] // 4,
           "mask": {"size": z["chunk"]}, "rot": {"dims": d // 2, "base": 10000.0}, "scale": d ** -0.5}
    par = {"left": {"heads": z["heads"], "kv_heads": z["kv"], "dim": d, "vdim": d, "scale": d ** -0.5,
                    "mask": {"size": z["chunk"] // 2, "keep_first": 64}, "rot": {"dims": d, "base": 1.0e6}},
           "right": {"heads": z["width"] // 64 // 2, "dim": 64, "decay_rank": 64}, "left_scale": 0.5, "right_scale": 1.0}
    dense = {"kind": "dense", "ff": z["ff"] * 2 // 3 // 64 * 64}        # (gated: three matrices instead of two)
    layers = []
    for i in range(repeats):
        layers += [{"type": "latent_attention", "mixer": dict(lat), "mlp": dense},
                   {"type": "parallel", "mixer": par, "mlp": dense},
                   {"type": "latent_attention", "mixer": dict(lat, kv_from=3 * i), "mlp": dense}]
    return SisavikConfig.from_dict({"architecture": "Sisavik", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
                                    "canon": {"taps": 4}, "layers": layers})


def kagolix_dense_config(z: dict, repeats: int = 2) -> KagolixConfig:
    """The Kagolix stack a Sisavik stack is measured against: the same mixers as ``hybrid_config`` with a
    dense feed-forward in every layer (Sisavik has no experts)."""
    cfg = hybrid_config(z, repeats).to_dict()
    for l in cfg["layers"]:
        l["mlp"] = {"kind": "dense", "ff": z["ff"]}
    return KagolixConfig.from_dict(cfg)


def gizezen_config(z: dict, repeats: int = 3) -> GizezenConfig:
    """Pairs of sliding-window attention layers, the second reading the first one's keys and values, each
    with routed experts and a shared expert: head sizes, window, taps and expert sizes of the order real
    models use."""
    d = z["dim"]
    att = {"heads": z["heads"], "kv_heads": z["kv"], "dim": d, "vdim": d, "conv": 4, "mask": {"size": z["chunk"]},
           "rot": {"dims": d, "base": 5.0e5, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}},
           "scale": d ** -0.5}
    moe = {"kind": "moe", "expert": {"ff": z["eff"]}, "router": {"experts": z["experts"], "top": z["top"]},
           "shared": {"ff": z["eff"]}}
    layers = []
    for i in range(repeats):
        layers += [{"type": "attention", "mixer": dict(att), "mlp": moe},
                   {"type": "attention", "mixer": dict(att, kv_from=2 * i), "mlp": moe}]
    return GizezenConfig.from_dict({"architecture": "Gizezen", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
                                    "residual_mult": 0.6, "embedding": {"scale": 1.5}, "layers": layers})


def lopilix_config(z: dict, times: int = 2, streams: int = 4) -> LopilixConfig:
    """Differential attention with a dense feed-forward, HGRN2 with experts, latent attention with experts; the
    three layers run ``times`` times in a row on the same weights (six layer runs), over ``streams`` residual
    streams.  Head sizes, ranks and expert sizes of the order real models use."""
    d = z["dim"]
    att = {"heads": z["heads"], "kv_heads": z["kv"], "dim": d // 2, "vdim": d, "rot": {"dims": d // 2, "base": 5.0e5},
           "scale": (d // 2) ** -0.5, "diff": 0.2}
    rec = {"heads": z["width"] // d, "dim": d, "vdim": d}
    lat = {"heads": z["heads"], "dim": d // 2, "rot_dim": d // 2, "vdim": d, "kv_rank": 4 * d, "scale": d ** -0.5,
           "rot": {"dims": d // 2, "base": 5.0e5, "scaling": {"factor": 8.0, "original": 4096, "fast": 16.0, "slow": 2.0}}}
    dense = {"kind": "dense", "ff": z["ff"] * 2 // 3 // 64 * 64}        # (gated: three matrices instead of two)
    moe = {"kind": "moe", "expert": {"ff": z["eff"]},
           "router": {"experts": z["experts"], "top": z["top"], "scale": 2.0, "groups": {"count": z["experts"] // 2, "keep": z["experts"] // 4}}}
    layers = [{"type": "attention", "mixer": att, "mlp": dense}, {"type": "hgrn2", "mixer": rec, "mlp": moe},
              {"type": "latent_attention", "mixer": lat, "mlp": moe}]
    return LopilixConfig.from_dict({"architecture": "Lopilix", "width": z["width"], "vocab": z["vocab"], "norm": {"eps": 1e-6},
                                    "residual_mult": 0.5, "streams": streams, "logit_scale": 0.5, "max_positions": 8192,
                                    "loop": {"start": 0, "stop": 3, "times": times}, "layers": layers})


def kagolix_attention_moe_config(z: dict, n_layers: int = 6) -> KagolixConfig:
    """The Kagolix stack a Gizezen stack is measured against: chunk-local attention and routed experts in
    every layer (the same heads, head size, experts and expert width; no shared expert, no shared keys)."""
    att = {"type": "attention", "mixer": {"heads": z["heads"], "kv_heads": z["kv"], "dim": z["dim"], "vdim": z["dim"],
                                           "mask": {"size": z["chunk"]}, "scale": z["dim"] ** -0.5, "softcap": 30.0}}
    moe = {"kind": "moe", "expert": {"ff": z["eff"]}, "router": {"experts": z["experts"], "top": z["top"]}}
    return KagolixConfig.from_dict({"architecture": "Kagolix", "width": z["width"], "vocab": z["vocab"],
                                    "norm": {"eps": 1e-6, "groups": 2}, "logit_softcap": 30.0,
                                    "layers": [dict(att, mlp=moe) for _ in range(n_layers)]})


def dense_config(z: dict, n_layers: int) -> ModelConfig:
    cfg = ModelConfig(hidden_size=z["width"], intermediate_size=z["eff"], num_attention_heads=z["heads"],
                      num_key_value_heads=z["kv"], num_hidden_layers=n_layers, vocab_size=z["vocab"], rope_theta=1e6,
                      num_local_experts=z["experts"], num_experts_per_tok=z["top"], model_type="mixtral",
                      architectures=["MixtralForCausalLM"], explicit_head_dim=None)
    cfg.validate()
    return cfg


def synthetic_hybrid_store(cfg: KagolixConfig, device, dtype, seed: int = 0):
    """Random layer images generated on ``device`` and parked in pinned host memory: matrices
    ~ N(0, 0.02), norm weights near 1, small recurrence constants."""
    from ..runtime.weights import HostStore
    st = HostStore(cfg, dtype, pinned=torch.device(device).type == "cuda")
    g = torch.Generator(device=device).manual_seed(seed)
    for name in st.names:
        lay = st.layout(name)
        img = torch.zeros(lay.nbytes, dtype=torch.uint8, device=device)
        for k, v in lay.views(img, dtype).items():
            if cfg.family == "sisavik" and (k.startswith("norm") or k.startswith("canon")):
                v.copy_(0.1 * torch.randn(v.shape, generator=g, device=device))     # (stored around zero)
            elif cfg.family == "gizezen" and k.startswith("norm"):
                v[0].copy_(1.0 + 0.1 * torch.randn(v.shape[1:], generator=g, device=device))    # [weight; bias]
                v[1].copy_(0.1 * torch.randn(v.shape[1:], generator=g, device=device))
            elif cfg.family == "lopilix" and k.startswith("hc"):
                S = cfg.streams                                       # [in | out | mix]: an even read, a unit write, streams that keep themselves
                v.copy_(torch.cat([torch.full((S,), 1.0 / S), torch.ones(S), torch.eye(S).reshape(-1)]).to(device)
                        + 0.05 * torch.randn(v.shape, generator=g, device=device))
            elif k == "lower":
                v.copy_(0.9 * torch.rand(v.shape, generator=g, device=device))
            elif k.startswith("alpha"):
                v.fill_(0.5)
            elif k.startswith("norm") or k in ("qn", "kn", "mnorm", "dqn", "dkvn", "lqn", "lkn", "rnorm"):
                v.copy_(1.0 + 0.1 * torch.randn(v.shape, generator=g, device=device))
            elif k in ("r1", "r2"):
                v.copy_(torch.rand(v.shape, generator=g, device=device))       # (a negative r2 has no logarithm)
            elif k == "embed":
                v.copy_(torch.randn(v.shape, generator=g, device=device).to(v.dtype))
            elif v.dim() >= 2 and k != "conv":
                v.copy_((0.02 * torch.randn(v.shape, generator=g, device=device)).to(v.dtype))
            else:
                v.copy_(0.3 * torch.randn(v.shape, generator=g, device=device))
        st.alloc(name).copy_(img)
    return st


def _timed(fn, reps: int) -> float:
    fn()                                   # (the first call loads code objects and grows the allocator)
    torch.cuda.synchronize()
    t = time.perf_counter()
    for _ in range(reps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t) / reps


def bench_hybrid_model(z: dict, dtype, B: int, L: int, steps: int, dev, cfg=None, part="hybrid") -> dict:
    from ..engine import ShardedRunner
    from ..runtime.batch import StepEntry
    cfg = cfg if cfg is not None else hybrid_config(z)
    src = synthetic_hybrid_store(cfg, dev, dtype)
    r = ShardedRunner(cfg, src, device=dev, layer_num_per_shard=len(cfg.layer_names()), storage_location="cpu",
                      resident=True, token_budget=1 << 20, compute_dtype=dtype, state_tokens=B * (L + steps + 8),
                      state_seqs=B)
    rng = np.random.default_rng(0)
    toks = [rng.integers(0, cfg.vocab, L).tolist() for _ in range(B)]
    n = [0]

    def prefill(keep=False):
        n[0] += 1
        ids = [(n[0], b) for b in range(B)]
        r.step([StepEntry(i, t, [L - 1]) for i, t in zip(ids, toks)], [] if keep else ids)
        return ids
    prefill()
    t_pre = _timed(prefill, max(1, steps // 4))
    ids = prefill(keep=True)

    def decode():
        r.step([StepEntry(i, [7], [0]) for i in ids])
    decode()
    t_dec = _timed(decode, steps)
    out = {"part": part, "model": f"{cfg.family} {cfg.total_params() / 1e9:.2f}B params, {cfg.num_hidden_layers} layer runs, width {cfg.width}",
           "dtype": str(dtype), "batch": B, "context": L, "prefill_tok_s": B * L / t_pre, "prefill_ms": t_pre * 1e3,
           "decode_tok_s": B / t_dec, "decode_ms_per_step": t_dec * 1e3, "state_bytes": r.seq_cache.nbytes()}
    r.close()
    return out


def bench_dense_model(z: dict, n_layers: int, B: int, L: int, steps: int, dev) -> dict:
    from ..engine import ShardedRunner
    from ..runtime.weights import HostStore
    from ..utils.tokenizer import TokenizedPrompt
    cfg = dense_config(z, n_layers)
    src = HostStore.synthetic(cfg, dev, seed=0, fold_norms=True)
    r = ShardedRunner(cfg, src, device=dev, layer_num_per_shard=len(cfg.layer_names()), storage_location="cpu",
                      resident=True, token_budget=1 << 20, prefix_kv_cache=True, suffix_kv_cache=True,
                      prefix_attention="causal")
    rng = np.random.default_rng(0)
    pref = [rng.integers(3, cfg.vocab_size, L - 1).tolist() for _ in range(B)]
    sfx = [[5] for _ in range(B)]

    def tps():
        return [TokenizedPrompt(p, [list(s)], len(s), [len(s) - 1]) for p, s in zip(pref, sfx)]

    def prefill():
        r.prefix_cache = type(r.prefix_cache)(2 * cfg.num_key_value_heads * cfg.head_dim, r.dev, r.act_dtype, 8,
                                              suffix_reuse=True, host=False)
        r.run_tokenized(tps())
    prefill()
    t_pre = _timed(prefill, max(1, steps // 4))

    def decode():
        for s in sfx:
            s.append(7)
        r.run_tokenized(tps())
    decode()
    t_dec = _timed(decode, steps)
    out = {"part": "dense", "model": f"mixtral-structured {cfg.total_params() / 1e9:.2f}B params, {n_layers} layers, width {z['width']}",
           "dtype": "float16", "batch": B, "context": L, "prefill_tok_s": B * L / t_pre, "prefill_ms": t_pre * 1e3,
           "decode_tok_s": B / t_dec, "decode_ms_per_step": t_dec * 1e3}
    r.close()
    return out


def bench_kernels(z: dict, dtype, B: int, L: int, dev) -> dict:
    """Every hybrid kernel alone at the prefill shape (T = B L rows) and the decode shape (T = B rows at
    context L): seconds, and the fraction of the matrix peak (GEMM, attention) or of HBM bandwidth."""
    from ..ops import get_ops
    ops = get_ops(dev, dtype, family="hybrid")
    es = 2 if dtype == torch.bfloat16 else 4
    D, H, G, d = z["width"], z["heads"], z["kv"], z["dim"]
    res: Dict[str, dict] = {}

    def rec(name, sec, flops=0.0, nbytes=0.0):
        e = {"us": sec * 1e6}
        if flops:
            e["tflops"] = flops / sec / 1e12
            e["of_matrix_peak"] = flops / sec / PEAK_FLOPS
        if nbytes:
            e["gb_s"] = nbytes / sec / 1e9
            e["of_hbm"] = nbytes / sec / PEAK_BYTES
        res[name] = {k: round(v, 4) for k, v in e.items()}

    ps = 16
    for tag, lens, pos0 in (("prefill", [L] * B, [0] * B), ("decode", [1] * B, [L - 1] * B)):
        T = sum(lens)
        cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
        seq = np.repeat(np.arange(B), lens).astype(np.int32)
        pos = np.concatenate([np.arange(p, p + n) for p, n in zip(pos0, lens)]).astype(np.int32)
        npg = -(-(L + 1) // ps)
        table = np.arange(B * npg, dtype=np.int32).reshape(B, npg)
        meta = {k: torch.from_numpy(v).to(dev) for k, v in dict(
            tok_seq=seq, tok_pos=pos, cu=cu, pos0=np.asarray(pos0, np.int32), slot=np.arange(B, dtype=np.int32),
            page_table=table, kv_slot=(table[seq, pos // ps] * ps + pos % ps).astype(np.int32)).items()}
        meta["n_seqs"] = B
        if tag == "prefill":
            meta["q_tiles"] = torch.tensor([(b * L + o, min(128, L - o)) for b in range(B) for o in range(0, L, 128)],
                                           dtype=torch.int32, device=dev)
            meta["tile_cu"] = torch.arange(0, B * (-(-L // 128)) + 1, -(-L // 128), dtype=torch.int32, device=dev)
        reps = 5 if tag == "prefill" else 30
        x = torch.randn(T, D, device=dev)
        h = x.to(dtype)
        w = (0.02 * torch.randn(z["ff"], D, device=dev)).to(dtype)
        rec(f"{tag}/gemm {T}x{z['ff']}x{D}", _timed(lambda: ops.matmul_nt(h, w), reps), 2.0 * T * z["ff"] * D,
            es * (z["ff"] * D + T * D) + 4 * T * z["ff"])
        nw = torch.ones(D, device=dev)
        rec(f"{tag}/group_rmsnorm", _timed(lambda: ops.group_rmsnorm(x, nw, 2, 1e-6, dtype), reps), 0, T * D * (4 + es))
        y = torch.randn(T, D, device=dev)
        rec(f"{tag}/add_group_rmsnorm", _timed(lambda: ops.add_group_rmsnorm_(x, y, nw, 2, 1e-6), reps), 0, T * D * 12)
        kc = torch.randn(B * npg, ps, G * d, device=dev).to(dtype)
        vc = torch.randn(B * npg, ps, G * d, device=dev).to(dtype)
        q = torch.randn(T, H * d, device=dev).to(dtype)
        r1 = torch.rand(H, device=dev)
        keys = float(np.mean([p % z["chunk"] + 1 for p in pos]))
        rec(f"{tag}/attention", _timed(lambda: ops.attn_paged(q, kc, vc, meta, H, G, d, d, d ** -0.5, 30.0, r1, r1,
                                                                 z["chunk"], ps, dtype), reps),
            4.0 * T * keys * H * d, 0 if tag == "prefill" else 2.0 * B * keys * G * d * es)
        Wd = z["width"]
        u = torch.randn(T, Wd, device=dev)
        g = torch.randn(T, 2 * Wd, device=dev)
        st = torch.zeros(B, Wd, device=dev)
        lam = torch.randn(Wd, device=dev)
        rec(f"{tag}/rglru_scan", _timed(lambda: ops.rglru_scan(u, g, lam, u, st, meta, 8.0, dtype), reps), 0,
            T * Wd * (16 + es))
        cw, cb = torch.randn(Wd, 4, device=dev), torch.randn(Wd, device=dev)
        cst = torch.zeros(B, 3, Wd, device=dev)
        rec(f"{tag}/causal_conv", _timed(lambda: ops.causal_conv(u, cw, cb, cst, meta), reps), 0, T * Wd * 8)
        nh, P, N = z["mh"], z["mp"], z["state"]
        xbc = torch.randn(T, nh * P + 2 * N, device=dev)
        zz = torch.randn(T, nh * P, device=dev)
        dt = torch.randn(T, nh, device=dev)
        hp = torch.randn(nh, device=dev)
        sst = torch.zeros(B, nh, N, P, device=dev)
        rec(f"{tag}/ssd_scan", _timed(lambda: ops.ssd_scan(xbc, zz, dt, hp, hp * 0.3, hp, sst, meta, nh, P, N, 1), reps),
            6.0 * T * nh * P * N, (T * nh * P * 12) if tag == "prefill" else 8.0 * B * nh * N * P)
    # the dense family's like kernels (fp16): GEMM at the prefill and decode shapes, RMSNorm
    dops = get_ops(dev)
    for tag, T in (("prefill", B * L), ("decode", B)):
        h16 = torch.randn(T, D, device=dev).half()
        w16 = (0.02 * torch.randn(z["ff"], D, device=dev)).half()
        reps = 5 if tag == "prefill" else 30
        rec(f"dense {tag}/gemm {T}x{z['ff']}x{D}", _timed(lambda: dops.gemm(h16, w16), reps), 2.0 * T * z["ff"] * D,
            2 * (z["ff"] * D + T * D + T * z["ff"]))
        nw16 = torch.ones(D, device=dev).half()
        rec(f"dense {tag}/rmsnorm", _timed(lambda: dops.rmsnorm(h16, nw16, 1e-6), reps), 0, T * D * 4)
    return {"part": "kernels", "dtype": str(dtype), "batch": B, "context": L, "kernels": res}


def step_meta(B: int, lens, pos0, L: int, dev, ps: int = 16) -> dict:
    """Device metadata of a step of B requests (rows ``lens`` from positions ``pos0``) whose pages are
    laid out request after request."""
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    seq = np.repeat(np.arange(B), lens).astype(np.int32)
    pos = np.concatenate([np.arange(p, p + n) for p, n in zip(pos0, lens)]).astype(np.int32)
    npg = -(-(L + 1) // ps)
    table = np.arange(B * npg, dtype=np.int32).reshape(B, npg)
    meta = {k: torch.from_numpy(v).to(dev) for k, v in dict(
        tok_seq=seq, tok_pos=pos, cu=cu, pos0=np.asarray(pos0, np.int32), slot=np.arange(B, dtype=np.int32),
        page_table=table, kv_slot=(table[seq, pos // ps] * ps + pos % ps).astype(np.int32)).items()}
    meta.update(n_seqs=B, n_pages=B * npg, pos_host=pos)
    if max(lens) >= 16:
        from ..runtime.batch import Q_TILE_ROWS as QT
        meta["q_tiles"] = torch.tensor([(int(a) + o, min(QT, int(b) - int(a) - o)) for a, b in zip(cu[:-1], cu[1:])
                                        for o in range(0, int(b) - int(a), QT)], dtype=torch.int32, device=dev)
        meta["tile_cu"] = torch.tensor(np.concatenate([[0], np.cumsum([-(-int(n) // QT) for n in lens])]), dtype=torch.int32,
                                       device=dev)
        if all(p == 0 for p in pos0):
            meta["local_table"] = torch.from_numpy((cu[:-1, None] + np.arange(max(lens), dtype=np.int32)[None, :]).astype(np.int32)).to(dev)
    return meta


def bench_sisavik_kernels(z: dict, dtype, B: int, L: int, dev) -> dict:
    """The kernels of the Sisavik mixers alone at the prefill shape (T = B L rows) and the decode shape
    (B rows at context L), each beside the like kernel of the Kagolix family on a like shape."""
    from ..models.sisavik import DECAY_SCALE
    from ..ops import get_ops
    ops = get_ops(dev, dtype, family="hybrid")
    es = 2 if dtype == torch.bfloat16 else 4
    cfg = sisavik_config(z, 1)
    lat, par = cfg.layers[0].mixer, cfg.layers[1].mixer
    D, ps = z["width"], 16
    res: Dict[str, dict] = {}

    def rec(name, sec, flops=0.0, nbytes=0.0):
        e = {"us": sec * 1e6}
        if flops:
            e["tflops"] = flops / sec / 1e12
            e["of_matrix_peak"] = flops / sec / PEAK_FLOPS
        if nbytes:
            e["gb_s"] = nbytes / sec / 1e9
            e["of_hbm"] = nbytes / sec / PEAK_BYTES
        res[name] = {k: round(v, 4) for k, v in e.items()}

    for tag, lens, pos0 in (("prefill", [L] * B, [0] * B), ("decode", [1] * B, [L - 1] * B)):
        T = sum(lens)
        meta = step_meta(B, lens, pos0, L, dev, ps)
        pos = meta["pos_host"]
        reps = 5 if tag == "prefill" else 30
        # sigmoid-gated window attention with kept tokens (left mixer) | Kagolix: chunk-local softmax attention
        a = par["left"]
        H, G, d = a["heads"], a["kv_heads"], a["dim"]
        win, keep = a["mask"]["size"], a["mask"]["keep_first"]
        kc = torch.randn(meta["n_pages"], ps, G * d, device=dev).to(dtype)
        vc = torch.randn(meta["n_pages"], ps, G * d, device=dev).to(dtype)
        q = torch.randn(T, H * d, device=dev)
        gb = torch.randn(H, device=dev)
        keys = float(np.mean([min(p + 1, win) + min(keep, max(0, p - win + 1)) for p in pos]))
        rec(f"{tag}/gated window attention", _timed(lambda: ops.attn_paged(
            q, kc, vc, meta, H, G, d, d, d ** -0.5, 0.0, None, None, 0, ps, dtype, window=win, keep_first=keep, gate_bias=gb,
            out_scale=0.5), reps), 4.0 * T * keys * H * d, 0 if tag == "prefill" else 2.0 * B * keys * G * d * es)
        qk = q.to(dtype)
        r1 = torch.rand(H, device=dev)
        keys_k = float(np.mean([p % z["chunk"] + 1 for p in pos]))
        rec(f"kagolix {tag}/chunk attention", _timed(lambda: ops.attn_paged(qk, kc, vc, meta, H, G, d, d, d ** -0.5, 30.0, r1, r1,
                                                                              z["chunk"], ps, dtype), reps),
            4.0 * T * keys_k * H * d, 0 if tag == "prefill" else 2.0 * B * keys_k * G * d * es)
        # latent attention: one key / value head of latent rows, all query heads (the folded form)
        r, dr, Hl, wl = lat["kv_rank"], lat["rot_dim"], lat["heads"], lat["mask"]["size"]
        pool = torch.randn(meta["n_pages"], ps, r + dr, device=dev).to(dtype)
        qa = torch.randn(T, Hl * (r + dr), device=dev)
        keys_l = float(np.mean([min(p + 1, wl) for p in pos]))
        if tag == "decode":
            rec(f"{tag}/latent attention (folded)", _timed(lambda: ops.attn_paged(
                qa, pool, pool, meta, Hl, 1, r + dr, r, d ** -0.5, 0.0, None, None, 0, ps, dtype, window=wl), reps),
                2.0 * T * keys_l * Hl * (2 * r + dr), 2.0 * B * keys_l * (r + dr) * es)
        else:
            dl, dvl = lat["dim"] + dr, lat["vdim"]
            kf = torch.randn(T, Hl * dl, device=dev).to(dtype)
            vf = torch.randn(T, Hl * dvl, device=dev).to(dtype)
            ql = torch.randn(T, Hl * dl, device=dev)
            lm = dict(meta, page_table=meta["local_table"])
            rec(f"{tag}/latent attention (keys and values unfolded)", _timed(lambda: ops.attn_paged(
                ql, kf.view(T, 1, -1), vf.view(T, 1, -1), lm, Hl, Hl, dl, dvl, d ** -0.5, 0.0, None, None, 0, 1, dtype,
                window=wl), reps), 2.0 * T * keys_l * Hl * (dl + dvl))
        # delta rule | Kagolix: state-space scan
        rr = par["right"]
        Hr, dd = rr["heads"], rr["dim"]
        zz = torch.randn(T, 6 * Hr * dd, device=dev)
        cols = [zz[:, i * Hr * dd:(i + 1) * Hr * dd] for i in range(6)]
        w0, nw = torch.randn(Hr * dd, device=dev), torch.ones(Hr * dd, device=dev)
        st = torch.zeros(B, Hr, dd, dd, device=dev)
        o = torch.empty(T, Hr * dd, device=dev, dtype=dtype)
        rec(f"{tag}/delta rule", _timed(lambda: ops.delta_rule_scan(*cols, w0, nw, st, meta, Hr, dd, decay_scale=DECAY_SCALE,
                                                                      key_eps=1e-6, norm_eps=1e-6, out_scale=1.0, out=o), reps),
            10.0 * T * Hr * dd * dd, (T * Hr * dd * (24 + es)) if tag == "prefill" else 8.0 * B * Hr * dd * dd)
        nh, P, N = z["mh"], z["mp"], z["state"]
        xbc = torch.randn(T, nh * P + 2 * N, device=dev)
        z2, dt, hp = torch.randn(T, nh * P, device=dev), torch.randn(T, nh, device=dev), torch.randn(nh, device=dev)
        sst = torch.zeros(B, nh, N, P, device=dev)
        rec(f"kagolix {tag}/ssd_scan", _timed(lambda: ops.ssd_scan(xbc, z2, dt, hp, hp * 0.3, hp, sst, meta, nh, P, N, 1), reps),
            6.0 * T * nh * P * N, (T * nh * P * 12) if tag == "prefill" else 8.0 * B * nh * N * P)
        # input convolution (+ input, cast) | Kagolix: causal convolution; norms; gate product; head norm + rotation + page write
        x = torch.randn(T, D, device=dev)
        cw, cb = torch.randn(D, 4, device=dev) * 0.1, torch.zeros(D, device=dev)
        cst = torch.zeros(B, 3, D, device=dev)
        rec(f"{tag}/input convolution", _timed(lambda: ops.causal_conv(x, cw, None, cst, meta, residual=True, out_dtype=dtype), reps),
            0, T * D * (4 + es))
        rec(f"kagolix {tag}/causal_conv", _timed(lambda: ops.causal_conv(x, cw, cb, cst, meta), reps), 0, T * D * 8)
        y, nwd = torch.randn(T, D, device=dev), torch.zeros(D, device=dev)
        rec(f"{tag}/post-norm + residual add", _timed(lambda: ops.add_group_rmsnorm_(x, y, nwd, 1, 1e-6, w_offset=1.0), reps), 0, T * D * 12)
        rec(f"kagolix {tag}/post-norm + residual add", _timed(lambda: ops.add_group_rmsnorm_(x, y, nwd + 1, 2, 1e-6), reps), 0, T * D * 12)
        ff = cfg.layers[0].mlp["ff"]
        gu = torch.randn(T, 2 * ff, device=dev)
        rec(f"{tag}/gelu gate product", _timed(lambda: ops.gate_mul(gu, dtype, "gelu_tanh"), reps), 0, T * ff * (8 + es))
        rec(f"kagolix {tag}/silu gate product", _timed(lambda: ops.gate_mul(gu, dtype, "silu"), reps), 0, T * ff * (8 + es))
        zq = torch.randn(T, (H + G) * d, device=dev)
        qn = torch.ones(d, device=dev)
        rec(f"{tag}/key norm + rotation + page write", _timed(lambda: ops.head_norm_rope(
            zq, G, d, H * d, d, kc.view(-1, G * d), 0, d, meta, w=qn, eps=1e-6, rot=(d, 1e6), row_map=meta["kv_slot"],
            raw=vc.view(-1, G * d)), reps), 0, T * G * d * (4 + 2 * es))
        kn = torch.ones(G * d, device=dev)
        rec(f"kagolix {tag}/key norm + page write", _timed(lambda: ops.kv_store(zq[:, H * d:], kn, 1e-6, zq[:, H * d:], kc, vc,
                                                                                 meta["kv_slot"]), reps), 0, T * G * d * (8 + 2 * es))
        h = x.to(dtype)
        w = (0.02 * torch.randn(2 * ff, D, device=dev)).to(dtype)
        rec(f"{tag}/gemm {T}x{2 * ff}x{D}", _timed(lambda: ops.matmul_nt(h, w), reps), 4.0 * T * ff * D,
            es * (2 * ff * D + T * D) + 8 * T * ff)
    return {"part": "kernels", "family": "sisavik", "dtype": str(dtype), "batch": B, "context": L, "kernels": res}


def bench_gizezen_kernels(z: dict, dtype, B: int, L: int, dev) -> dict:
    """The kernels of a Gizezen layer alone at the prefill shape (T = B L rows) and the decode shape (B rows
    at context L), each beside the like kernel of the Kagolix family on a like shape."""
    from ..models.gizezen import SINK_SCORE, _rot
    from ..ops import get_ops
    ops = get_ops(dev, dtype, family="hybrid")
    es = 2 if dtype == torch.bfloat16 else 4
    cfg = gizezen_config(z, 1)
    m, mlp = cfg.layers[0].mixer, cfg.layers[0].mlp
    D, ps = z["width"], 16
    H, G, d, win, taps = m["heads"], m["kv_heads"], m["dim"], m["mask"]["size"], m["conv"]
    E, top, ff = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
    res: Dict[str, dict] = {}

    def rec(name, sec, flops=0.0, nbytes=0.0):
        e = {"us": sec * 1e6}
        if flops:
            e["tflops"] = flops / sec / 1e12
            e["of_matrix_peak"] = flops / sec / PEAK_FLOPS
        if nbytes:
            e["gb_s"] = nbytes / sec / 1e9
            e["of_hbm"] = nbytes / sec / PEAK_BYTES
        res[name] = {k: round(v, 4) for k, v in e.items()}

    for tag, lens, pos0 in (("prefill", [L] * B, [0] * B), ("decode", [1] * B, [L - 1] * B)):
        T = sum(lens)
        meta = step_meta(B, lens, pos0, L, dev, ps)
        meta["max_rows"] = max(lens)
        pos = meta["pos_host"]
        reps = 5 if tag == "prefill" else 30
        # window attention with the silent softmax entry and head gates | Kagolix: chunk-local softmax attention
        kc = torch.randn(meta["n_pages"], ps, G * d, device=dev).to(dtype)
        vc = torch.randn(meta["n_pages"], ps, G * d, device=dev).to(dtype)
        q = torch.randn(T, H * d, device=dev)
        zz = torch.randn(T, (H + 2 * G) * d + H, device=dev)
        hg = zz[:, (H + 2 * G) * d:]
        keys = float(np.mean([min(p + 1, win) for p in pos]))
        rec(f"{tag}/window attention, silent entry, head gates", _timed(lambda: ops.attn_paged(
            q, kc, vc, meta, H, G, d, d, d ** -0.5, 0.0, None, None, 0, ps, dtype, window=win, sink=SINK_SCORE, head_gate=hg), reps),
            4.0 * T * keys * H * d, 0 if tag == "prefill" else 2.0 * B * keys * G * d * es)
        qk = q.to(dtype)
        r1 = torch.rand(H, device=dev)
        keys_k = float(np.mean([p % z["chunk"] + 1 for p in pos]))
        rec(f"kagolix {tag}/chunk attention", _timed(lambda: ops.attn_paged(qk, kc, vc, meta, H, G, d, d, d ** -0.5, 30.0, r1, r1,
                                                                              z["chunk"], ps, dtype), reps),
            4.0 * T * keys_k * H * d, 0 if tag == "prefill" else 2.0 * B * keys_k * G * d * es)
        # convolution of q | k | v, rotation, unit norm, page write | Kagolix: query norm, key norm + page write
        C = (H + 2 * G) * d
        cw = torch.randn(C, taps, device=dev) * 0.3
        cst = torch.zeros(B, taps - 1, C, device=dev)
        qo = torch.empty(T, H * d, device=dev)
        rot = _rot(m)

        def qkv_path():
            ops.qkv_conv_rope_store(zz, cw, cst, meta, H, G, d, d, qo, kc, vc, eps=1e-6, rot=rot)
        rec(f"{tag}/q k v convolution + rotation + unit norm + page write", _timed(qkv_path, reps), 0,
            T * (C * 4 + H * d * 4 + 2 * G * d * es))
        kn, qn = torch.ones(G * d, device=dev), torch.ones(H * d, device=dev)

        def kagolix_qkv():
            ops.group_rmsnorm(zz[:, :H * d], qn, 1, 1e-6, out_dtype=dtype)
            ops.kv_store(zz[:, H * d:(H + G) * d], kn, 1e-6, zz[:, (H + G) * d:C], kc, vc, meta["kv_slot"])
        rec(f"kagolix {tag}/query norm, key norm + page write", _timed(kagolix_qkv, reps), 0, T * (C * 4 + (H + 2 * G) * d * es))
        # norms and residual updates
        x, y = torch.randn(T, D, device=dev), torch.randn(T, D, device=dev)
        wb, al = torch.randn(2, D, device=dev), torch.tensor([0.5], device=dev)
        rec(f"{tag}/dyt norm", _timed(lambda: ops.dyt_norm(x, wb, al, dtype), reps), 0, T * D * (4 + es))
        nw = torch.ones(D, device=dev)
        rec(f"kagolix {tag}/group norm", _timed(lambda: ops.group_rmsnorm(x, nw, 2, 1e-6, dtype), reps), 0, T * D * (4 + es))
        rec(f"{tag}/residual add + dyt norm", _timed(lambda: ops.add_scaled_dyt_norm_(x, y, 0.6, wb, al, dtype), reps), 0,
            T * D * (12 + es))

        def kagolix_add_norm():
            ops.add_group_rmsnorm_(x, y, nw, 2, 1e-6)
            ops.group_rmsnorm(x, nw, 2, 1e-6, dtype)
        rec(f"kagolix {tag}/post-norm + residual add, group norm", _timed(kagolix_add_norm, reps), 0, T * D * (16 + es))
        # routing and the experts' combine
        zr = torch.randn(T, E + 1, device=dev)
        logits = zr[:, :E]
        rec(f"{tag}/top-k routing", _timed(lambda: ops.moe_route_topk(logits, top), reps), 0, T * (E * 4 + top * 20))
        corr = torch.zeros(E, device=dev)
        rec(f"kagolix {tag}/corrected routing", _timed(lambda: ops.moe_route_corrected(logits, corr, top), reps), 0,
            T * (E * 4 + top * 20))
        route = ops.moe_route_topk(logits, top)
        yo, ys = torch.randn(T * top, D, device=dev), torch.randn(T, D, device=dev)
        rec(f"{tag}/expert sum + gated shared expert + residual add", _timed(
            lambda: ops.moe_combine_(x, yo, route, 0.6, ys, zr[:, E:]), reps), 0, T * D * 4 * (top + 3))

        def kagolix_combine():
            ops.add_group_rmsnorm_(x, ops.moe_weighted_sum(yo, route), nw, 2, 1e-6)
        rec(f"kagolix {tag}/expert sum, post-norm + residual add", _timed(kagolix_combine, reps), 0, T * D * 4 * (top + 5))
        gu = torch.randn(T * top, 2 * ff, device=dev)
        rec(f"{tag}/silu gate product", _timed(lambda: ops.gate_mul(gu, dtype, "silu"), reps), 0, T * top * ff * (8 + es))
        h = x.to(dtype)
        n_in = C + H
        w = (0.02 * torch.randn(n_in, D, device=dev)).to(dtype)
        rec(f"{tag}/gemm {T}x{n_in}x{D}", _timed(lambda: ops.matmul_nt(h, w), reps), 2.0 * T * n_in * D,
            es * (n_in * D + T * D) + 4 * T * n_in)
    return {"part": "kernels", "family": "gizezen", "dtype": str(dtype), "batch": B, "context": L, "kernels": res}


def bench_lopilix_kernels(z: dict, dtype, B: int, L: int, dev) -> dict:
    """The kernels of the Lopilix layers alone at the prefill shape (T = B L rows) and the decode shape (B rows at
    context L), each beside the like kernel of the Kagolix family on a like shape."""
    from ..models.lopilix import _rot
    from ..ops import get_ops
    ops = get_ops(dev, dtype, family="hybrid")
    es = 2 if dtype == torch.bfloat16 else 4
    cfg = lopilix_config(z, 1)
    att, rc, lat = (l.mixer for l in cfg.layers)
    mlp = cfg.layers[1].mlp
    D, S, ps = z["width"], cfg.streams, 16
    H, G, d, dv = att["heads"], att["kv_heads"], att["dim"], att["vdim"]
    E, top, ff = mlp["router"]["experts"], mlp["router"]["top"], mlp["expert"]["ff"]
    res: Dict[str, dict] = {}

    def rec(name, sec, flops=0.0, nbytes=0.0):
        e = {"us": sec * 1e6}
        if flops:
            e["tflops"] = flops / sec / 1e12
            e["of_matrix_peak"] = flops / sec / PEAK_FLOPS
        if nbytes:
            e["gb_s"] = nbytes / sec / 1e9
            e["of_hbm"] = nbytes / sec / PEAK_BYTES
        res[name] = {k: round(v, 4) for k, v in e.items()}

    for tag, lens, pos0 in (("prefill", [L] * B, [0] * B), ("decode", [1] * B, [L - 1] * B)):
        T = sum(lens)
        meta = step_meta(B, lens, pos0, L, dev, ps)
        meta["max_rows"] = max(lens)
        pos = meta["pos_host"]
        reps = 5 if tag == "prefill" else 30
        keys = float(np.mean([p + 1 for p in pos]))
        # two score maps over shared values (2 H heads over 2 G key heads, fp32 out) | Kagolix: chunk-local softmax attention
        kc = torch.randn(meta["n_pages"], ps, 2 * G * d, device=dev).to(dtype)
        vc = torch.randn(meta["n_pages"], ps, G * dv, device=dev).to(dtype)
        q = torch.randn(T, 2 * H * d, device=dev)
        a = torch.empty(T, 2 * H * dv, device=dev)
        rec(f"{tag}/differential attention, two maps", _timed(lambda: ops.attn_paged(
            q, kc, vc, meta, 2 * H, 2 * G, d, dv, d ** -0.5, 0.0, None, None, 0, ps, dtype, out=a, v_heads=G), reps),
            2.0 * T * keys * 2 * H * (d + dv), 0 if tag == "prefill" else B * keys * (2 * G * d + G * dv) * es)
        dk = z["dim"]
        kk = torch.randn(meta["n_pages"], ps, G * dk, device=dev).to(dtype)
        qk = torch.randn(T, H * dk, device=dev).to(dtype)
        r1 = torch.rand(H, device=dev)
        keys_k = float(np.mean([p % z["chunk"] + 1 for p in pos]))
        rec(f"kagolix {tag}/chunk attention", _timed(lambda: ops.attn_paged(qk, kk, kk, meta, H, G, dk, dk, dk ** -0.5, 30.0, r1, r1,
                                                                              z["chunk"], ps, dtype), reps),
            4.0 * T * keys_k * H * dk, 0 if tag == "prefill" else 2.0 * B * keys_k * G * dk * es)
        lam = 0.1 * torch.randn(4, d, device=dev)
        rec(f"{tag}/differential combine + unit norm", _timed(lambda: ops.diff_combine(a, lam, 0.2, H, dv, 1e-6, dtype), reps), 0,
            T * H * dv * (8 + es))
        # q and k: norm per head and map, rotation, page write; v: page write | Kagolix: query norm, key norm + page write
        C = 2 * H * d + 2 * G * d + G * dv
        zz = torch.randn(T, C + D, device=dev)
        qn = torch.ones(d, device=dev)
        qo = torch.empty(T, 2 * H * d, device=dev)
        rot = _rot(att)

        def qkv_path():
            ops.qkv_conv_rope_store(zz, None, None, meta, 2 * H, 2 * G, d, dv, qo, kc, vc, eps=1e-6, rot=rot, v_heads=G, q_norm=qn, k_norm=qn)
        rec(f"{tag}/q k norm + rotation, k v page write", _timed(qkv_path, reps), 0, T * (C * 4 + 2 * H * d * 4 + (2 * G * d + G * dv) * es))
        Ck = (H + 2 * G) * dk
        zk = torch.randn(T, Ck, device=dev)
        knw, qnw = torch.ones(G * dk, device=dev), torch.ones(H * dk, device=dev)

        def kagolix_qkv():
            ops.group_rmsnorm(zk[:, :H * dk], qnw, 1, 1e-6, out_dtype=dtype)
            ops.kv_store(zk[:, H * dk:(H + G) * dk], knw, 1e-6, zk[:, (H + G) * dk:Ck], kk, kk, meta["kv_slot"])
        rec(f"kagolix {tag}/query norm, key norm + page write", _timed(kagolix_qkv, reps), 0, T * (Ck * 4 + (H + 2 * G) * dk * es))
        # the residual streams
        xs, y = torch.randn(T, S * D, device=dev), torch.randn(T, D, device=dev)
        hc = torch.cat([torch.full((S,), 1.0 / S), torch.ones(S), torch.eye(S).reshape(-1)]).to(dev)
        nw = torch.ones(D, device=dev)
        gate = zz[:, C:C + D]
        rec(f"{tag}/streams sum + norm", _timed(lambda: ops.streams_norm(xs, hc, nw, 1e-6, dtype, S), reps), 0, T * D * (4 * S + es))
        rec(f"{tag}/streams update, gated", _timed(lambda: ops.streams_update_(xs, y, gate, hc, 0.5, S), reps), 0, T * D * 4 * (2 * S + 2))
        rec(f"{tag}/streams update, gated + next norm", _timed(lambda: ops.streams_update_norm_(xs, y, gate, hc, 0.5, S, hc, nw, 1e-6, dtype), reps),
            0, T * D * (4 * (2 * S + 2) + es))
        x = torch.randn(T, D, device=dev)
        rec(f"kagolix {tag}/group norm", _timed(lambda: ops.group_rmsnorm(x, nw, 2, 1e-6, dtype), reps), 0, T * D * (4 + es))

        def kagolix_add_norm():
            ops.add_group_rmsnorm_(x, y, nw, 2, 1e-6)
            ops.group_rmsnorm(x, nw, 2, 1e-6, dtype)
        rec(f"kagolix {tag}/post-norm + residual add, group norm", _timed(kagolix_add_norm, reps), 0, T * D * (16 + es))
        # the gated recurrence | Kagolix: the state-space scan
        Hr, dr, dvr = rc["heads"], rc["dim"], rc["vdim"]
        zr_ = torch.randn(T, 2 * Hr * dr + Hr * dvr, device=dev)
        lower, mn = 0.9 * torch.rand(Hr * dr, device=dev), torch.ones(dvr, device=dev)
        st = torch.zeros(B, Hr, dr, dvr, device=dev)
        rec(f"{tag}/hgrn2 scan + head norm", _timed(lambda: ops.hgrn2_scan(zr_[:, :Hr * dr], zr_[:, Hr * dr:2 * Hr * dr], zr_[:, 2 * Hr * dr:], None,
                                                                          lower, mn, st, meta, Hr, dr, dvr, 1e-6, dtype), reps),
            6.0 * T * Hr * dr * dvr, T * (zr_.shape[1] * 4 + Hr * dvr * (8 + es)) + 2 * B * Hr * dr * dvr * 4)
        nh, P, N = z["mh"], z["mp"], z["state"]
        xbc = torch.randn(T, nh * P + 2 * N, device=dev)
        z2, dt = torch.randn(T, nh * P, device=dev), torch.randn(T, nh, device=dev)
        hp = torch.rand(nh, device=dev)
        sst = torch.zeros(B, nh, N, P, device=dev)
        rec(f"kagolix {tag}/ssd_scan", _timed(lambda: ops.ssd_scan(xbc, z2, dt, hp, hp * 0.3, hp, sst, meta, nh, P, N, 1), reps),
            6.0 * T * nh * N * P, T * (xbc.shape[1] + 2 * nh * P + nh) * 4 + 2 * B * nh * N * P * 4)
        # latent attention: the folded form over latent rows, and keys and values made per head for whole prompts
        Hl, dn, drl, dvl, r = lat["heads"], lat["dim"], lat["rot_dim"], lat["vdim"], lat["kv_rank"]
        pool = torch.randn(meta["n_pages"], ps, r + drl, device=dev).to(dtype)
        qa = torch.randn(T, Hl * (r + drl), device=dev)
        if tag == "decode":
            rec(f"{tag}/latent attention (folded)", _timed(lambda: ops.attn_paged(
                qa, pool, pool, meta, Hl, 1, r + drl, r, lat["scale"], 0.0, None, None, 0, ps, dtype), reps),
                2.0 * T * keys * Hl * (2 * r + drl), B * keys * (r + drl) * es)
        else:
            kf = torch.randn(T, 1, Hl * (dn + drl), device=dev).to(dtype)
            vf = torch.randn(T, 1, Hl * dvl, device=dev).to(dtype)
            ql = torch.randn(T, Hl * (dn + drl), device=dev)
            al = torch.empty(T, Hl * dvl, device=dev)
            lm = dict(meta, page_table=meta["local_table"])
            rec(f"{tag}/latent attention (keys and values unfolded)", _timed(lambda: ops.attn_paged(
                ql, kf, vf, lm, Hl, Hl, dn + drl, dvl, lat["scale"], 0.0, None, None, 0, 1, dtype, out=al), reps),
                2.0 * T * keys * Hl * (dn + drl + dvl))
            g = torch.randn(T, Hl * dvl, device=dev)
            rec(f"{tag}/sigmoid output gate", _timed(lambda: ops.sigmoid_gate(al, g, dtype), reps), 0, T * Hl * dvl * (8 + es))
        # routing and the experts' activation
        zr = torch.randn(T, E + D, device=dev)
        logits = zr[:, :E]
        gr = mlp["router"]["groups"]
        rec(f"{tag}/grouped sigmoid routing", _timed(lambda: ops.moe_route_grouped(logits, top, gr["count"], gr["keep"], 2.0), reps), 0,
            T * (E * 4 + top * 20))
        corr = torch.zeros(E, device=dev)
        rec(f"kagolix {tag}/corrected routing", _timed(lambda: ops.moe_route_corrected(logits, corr, top), reps), 0,
            T * (E * 4 + top * 20))
        up = torch.randn(T * top, ff, device=dev)
        rec(f"{tag}/gelu (erf)", _timed(lambda: ops.unary(up, "gelu", dtype), reps), 0, T * top * ff * (4 + es))
        gu = torch.randn(T * top, 2 * ff, device=dev)
        rec(f"kagolix {tag}/silu gate product", _timed(lambda: ops.gate_mul(gu, dtype, "silu"), reps), 0, T * top * ff * (8 + es))
        route = ops.moe_route_grouped(logits, top, gr["count"], gr["keep"], 2.0)
        yo = torch.randn(T * top, D, device=dev)
        rec(f"{tag}/expert sum", _timed(lambda: ops.moe_weighted_sum(yo, route), reps), 0, T * D * 4 * (top + 1))
        h = torch.randn(T, D, device=dev).to(dtype)
        n_in = C + D
        w = (0.02 * torch.randn(n_in, D, device=dev)).to(dtype)
        rec(f"{tag}/gemm {T}x{n_in}x{D}", _timed(lambda: ops.matmul_nt(h, w), reps), 2.0 * T * n_in * D,
            es * (n_in * D + T * D) + 4 * T * n_in)
    return {"part": "kernels", "family": "lopilix", "dtype": str(dtype), "batch": B, "context": L, "kernels": res}


def main(a) -> int:
    """``bench.py --hybrid SIZE`` (one GPU)."""
    dev = torch.device("cuda", 0)
    torch.cuda.set_device(dev)
    z = SIZES[a.hybrid]
    dtype = torch.bfloat16 if a.hybrid_dtype == "bfloat16" else torch.float32
    B, L = a.hybrid_batch, a.hybrid_context
    lines: List[dict] = []
    parts = a.hybrid_parts.split(",")
    if getattr(a, "hybrid_family", "kagolix") == "lopilix":
        if "hybrid" in parts:
            lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev, lopilix_config(z), "lopilix"))
            print(json.dumps(lines[-1]), flush=True)
        if "dense" in parts:      # (the closest existing model: the Kagolix stack of attention, recurrent and state-space layers)
            lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev, hybrid_config(z), "kagolix"))
            print(json.dumps(lines[-1]), flush=True)
        if "kernels" in parts:
            lines.append(bench_lopilix_kernels(z, dtype, B, L, dev))
            print(json.dumps(lines[-1]), flush=True)
        if a.json_out:
            with open(a.json_out, "w") as f:
                json.dump(lines, f, indent=1)
        return 0
    if getattr(a, "hybrid_family", "kagolix") == "gizezen":
        if "hybrid" in parts:
            lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev, gizezen_config(z), "gizezen"))
            print(json.dumps(lines[-1]), flush=True)
        if "dense" in parts:      # (the closest existing model: a Kagolix stack of attention layers with experts)
            lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev, kagolix_attention_moe_config(z), "kagolix"))
            print(json.dumps(lines[-1]), flush=True)
        if "kernels" in parts:
            lines.append(bench_gizezen_kernels(z, dtype, B, L, dev))
            print(json.dumps(lines[-1]), flush=True)
        if a.json_out:
            with open(a.json_out, "w") as f:
                json.dump(lines, f, indent=1)
        return 0
    if getattr(a, "hybrid_family", "kagolix") == "sisavik":
        if "hybrid" in parts:
            lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev, sisavik_config(z), "sisavik"))
            print(json.dumps(lines[-1]), flush=True)
        if "dense" in parts:      # (the closest existing model here: a Kagolix stack of equal width, depth and ff)
            lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev, kagolix_dense_config(z), "kagolix"))
            print(json.dumps(lines[-1]), flush=True)
        if "kernels" in parts:
            lines.append(bench_sisavik_kernels(z, dtype, B, L, dev))
            print(json.dumps(lines[-1]), flush=True)
        if a.json_out:
            with open(a.json_out, "w") as f:
                json.dump(lines, f, indent=1)
        return 0
    if "hybrid" in parts:
        lines.append(bench_hybrid_model(z, dtype, B, L, a.steps * 8, dev))
        print(json.dumps(lines[-1]), flush=True)
    if "dense" in parts:
        lines.append(bench_dense_model(z, 6, B, L, a.steps * 8, dev))
        print(json.dumps(lines[-1]), flush=True)
    if "kernels" in parts:
        lines.append(bench_kernels(z, dtype, B, L, dev))
        print(json.dumps(lines[-1]), flush=True)
    if a.json_out:
        with open(a.json_out, "w") as f:
            json.dump(lines, f, indent=1)
    return 0
