"""Gizezen layer execution on packed weight images and packed step batches.

Every layer of a Gizezen stack is

    x <- x + m * mixer(N1(x));   x <- x + m * ff(N2(x))          (the second line only with an ff)

with x the fp32 residual stream, m = ``residual_mult`` and N a Dynamic Tanh norm: tanh(alpha x) w + b,
elementwise, without any statistic of the row.  The embedding rows enter the stream times
``embedding.scale``.  The mixer is grouped-query attention over a sliding window:

* one product gives [q | k | v | g] of the normed input; q, k and v then pass a short causal
  convolution per channel over the sequence (``conv`` taps, no bias; the last taps - 1 projected rows
  of a request are carried in its state slot);
* q and k are rotated in pairs (2i, 2i + 1) over the first ``rot.dims`` entries of a head, by angles
  pos * f_i whose frequencies may be rescaled by wavelength (``rot.scaling``), and then divided by
  their root mean square over the head; v is cached as convolved;
* p_j = exp(s_j) / (1 + sum exp(s)): the softmax has a silent entry of score 0 without a value;
* head h's output is multiplied by sigmoid(g_h), g = W_g N1(x), before the output projection;
* a layer with ``kv_from`` has no key / value projections and reads the named layer's cached keys and
  values with its own queries and window.

The feed-forward is a mixture of SiLU-gated experts: the ``top`` largest router logits choose, the
softmax over just those weighs; a shared expert, if the layer has one, is added times
sigmoid(W_sg h).  Each mechanism is an op of the backend (``ops/hip_seq.py``: the kernels of
``csrc/kernels/seq``; ``ops/torch_seq.py`` on the CPU) with its constants as arguments; this file only
strings them together.  Keys, values and convolution histories live in
:class:`~..runtime.seq_state.SequenceStateCache`.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .kagolix import HybridContext  # noqa: F401  (the context the engine builds for every hybrid family)
from .layout import LayerLayout, Placement, layer_kind, spec_layout, spec_placements

F32 = "f32"
SINK_SCORE = 0.0                   # the score of the softmax's silent entry
NO_WINDOW = 1 << 30                # a layer without a mask sees every earlier key


def _cols(m: dict):
    """(q, k, v) column counts of the stacked input projection; k = v = 0 for a layer that reads another's."""
    own = m.get("kv_from") is None
    return m["heads"] * m["dim"], (m["kv_heads"] * m["dim"]) if own else 0, (m["kv_heads"] * m["vdim"]) if own else 0


def _taps(m: dict) -> int:
    return int(m.get("conv") or 1)


def _window(m: dict) -> int:
    return int(m["mask"]["size"]) if m.get("mask") else 0


def _rot(m: dict):
    """(dims, base, scaling) of the pair rotation for ``head_norm_rope``, or None."""
    r = m.get("rot")
    if not r or int(r["dims"]) < 2:
        return None
    s = r.get("scaling")
    sc = (float(s["factor"]), float(s["low"]), float(s["high"]), float(s["original"])) if s else None
    return int(r["dims"]), float(r["base"]), sc


def _shared_ff(mlp: dict) -> int:
    return int(mlp["shared"]["ff"]) if mlp.get("shared") else 0


def _norm_specs(slot: str, alpha: str, tensor: str, D: int):
    return [(slot, (2, D), F32, [(tensor, 0, (D,)), (tensor + ".b", D, (D,))]),
            (alpha, (1,), F32, [(tensor + ".alpha", 0, ())])]


def _specs(cfg, name: str):
    """[(slot, shape, dtype tag, [(checkpoint tensor, element offset in the slot, shape)])]."""
    D, V = cfg.width, cfg.vocab
    kind = layer_kind(name)
    if kind == "embed":
        return [("embed", (V, D), None, [("embed", 0, (V, D))])]
    if kind == "head":
        return [("head", (V, D), None, [("head", 0, (V, D))])]
    if kind == "norm":
        return _norm_specs("norm", "alpha", "final.norm", D)
    L, p = cfg.layer(name), name + "."
    m, x = L.mixer, name + ".mix."
    qs, ks, vs = _cols(m)
    H, taps = m["heads"], _taps(m)
    proj, conv, at = [], [], 0
    for t, n in (("q", qs), ("k", ks), ("v", vs)):
        if n:
            proj.append((x + t, at * D, (n, D)))
            if "conv" in m:
                conv.append((x + t + ".conv", at * taps, (n, taps)))
            at += n
    proj.append((x + "g", at * D, (H, D)))
    out = _norm_specs("norm1", "alpha1", p + "norm1", D)
    out.append(("win", (at + H, D), None, proj))                       # [q; k; v; g]: one product
    if conv:
        out.append(("conv", (at, taps), F32, conv))
    out.append(("wo", (D, H * m["vdim"]), None, [(x + "o", 0, (D, H * m["vdim"]))]))
    if L.mlp is not None:
        y = p + "mlp."
        E, ff, fs = L.mlp["router"]["experts"], L.mlp["expert"]["ff"], _shared_ff(L.mlp)
        out += _norm_specs("norm2", "alpha2", p + "norm2", D)
        # [shared.gate; shared.up; router; shared.sg]: what every token needs of the feed-forward's input, one product
        wsr = [(y + "router", 2 * fs * D, (E, D))]
        if fs:
            wsr = [(y + "shared.gate", 0, (fs, D)), (y + "shared.up", fs * D, (fs, D))] + wsr + \
                  [(y + "shared.sg", (2 * fs + E) * D, (1, D))]
            out.append(("wsdown", (D, fs), None, [(y + "shared.down", 0, (D, fs))]))
        out.append(("wsr", (2 * fs + E + (1 if fs else 0), D), None, wsr))
        gu, dn = [], []
        for e in range(E):
            gu += [(f"{y}e{e}.gate", e * 2 * ff * D, (ff, D)), (f"{y}e{e}.up", (e * 2 + 1) * ff * D, (ff, D))]
            dn.append((f"{y}e{e}.down", e * D * ff, (D, ff)))
        out += [("wgu", (E, 2 * ff, D), None, gu), ("wdown", (E, D, ff), None, dn)]
    return out


def layout(cfg, name: str, elem_size: int = 2) -> LayerLayout:
    return spec_layout(layer_kind(name), _specs(cfg, name), elem_size)


def placements(cfg, name: str, elem_size: int = 2) -> List[Placement]:
    return spec_placements(layout(cfg, name, elem_size), _specs(cfg, name), elem_size)


def state_spec(cfg) -> dict:
    """What a request keeps between steps: per layer with keys and values of its own two page pools
    (a ``kv_from`` layer reads its owner's), per layer the last taps - 1 rows of its convolved
    projections, and every layer's window as a horizon behind which pages are given back."""
    paged, alias, slots, horizons = {}, {}, {}, []
    for i, l in enumerate(cfg.layers):
        name, m = f"l{i}", l.mixer
        if cfg.kv_owner(i) == i:
            paged[name] = {"k": m["kv_heads"] * m["dim"], "v": m["kv_heads"] * m["vdim"]}
        else:
            alias[name] = f"l{cfg.kv_owner(i)}"
        if _taps(m) > 1:
            slots[name] = {"conv": (_taps(m) - 1, sum(_cols(m)))}
        horizons.append(("window", _window(m) or NO_WINDOW, 0))
    return {"paged": paged, "alias": alias, "slots": slots, "horizons": horizons}


# ------------------------------------------------------------------------------------ execution
def _attention(ctx, m: dict, W, h, meta, name: str):
    ops, eps, cdt = ctx.ops, ctx.cfg.norm_eps, ctx.compute_dtype
    qs, ks, vs = _cols(m)
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    C = qs + ks + vs
    z = ops.matmul_nt(h, W["win"])                                        # fp32 [T, q | k | v | g]
    kc, vc = ctx.cache.kv(name)
    q = torch.empty(z.shape[0], qs, dtype=torch.float32, device=z.device)
    # convolution, rotation, unit norm and the write into the pages in one pass over the projected rows
    st = ctx.cache.recurrent(name)["conv"] if "conv" in W and _taps(m) > 1 else None
    ops.qkv_conv_rope_store(z, W.get("conv"), st, meta, H, G if ks else 0, d, dv, q, kc if ks else None, vc if ks else None,
                            eps=eps, rot=_rot(m))
    a = ops.attn_paged(q, kc, vc, meta, H, G, d, dv, scale=float(m["scale"]), softcap=0.0, r1=None, r2=None, chunk=0,
                       page_size=ctx.cache.page_size, out_dtype=cdt, window=_window(m), sink=SINK_SCORE,
                       head_gate=z[:, C:C + H])
    return ops.matmul_nt(a, W["wo"])


def _moe(ctx, mlp: dict, W, h, x):
    """x += m * (the chosen experts' weighted sum + the gated shared expert)."""
    ops, cdt = ctx.ops, ctx.compute_dtype
    E, top, fs = mlp["router"]["experts"], mlp["router"]["top"], _shared_ff(mlp)
    zr = ops.matmul_nt(h, W["wsr"])                                       # fp32 [T, shared gate | up | router | sg]
    route = ops.moe_route_topk(zr[:, 2 * fs:2 * fs + E], top)
    hp = ops.gather_rows(h, route.rows)                                   # rows sorted by expert
    gu = ops.grouped_matmul_nt(hp, W["wgu"], route.offs)                  # fp32 [T top, gate | up]
    yo = ops.grouped_matmul_nt(ops.silu_mul(gu, out_dtype=cdt), W["wdown"], route.offs)
    ys = gate = None
    if fs:
        ys = ops.matmul_nt(ops.silu_mul(zr[:, :2 * fs], out_dtype=cdt), W["wsdown"])
        gate = zr[:, 2 * fs + E:]
    return ops.moe_combine_(x, yo, route, ctx.cfg.residual_mult, ys, gate)


def run_block(ctx, W, x: torch.Tensor, meta: dict, name: str) -> torch.Tensor:
    cfg, ops, cdt = ctx.cfg, ctx.ops, ctx.compute_dtype
    L = cfg.layer(name)
    h = ops.dyt_norm(x, W["norm1"], W["alpha1"], cdt)
    y = _attention(ctx, L.mixer, W, h, meta, name)
    if L.mlp is None:
        return ops.add_scaled_(x, y, cfg.residual_mult)
    # (the residual update and the feed-forward's norm read and write the stream once)
    _moe(ctx, L.mlp, W, ops.add_scaled_dyt_norm_(x, y, cfg.residual_mult, W["norm2"], W["alpha2"], cdt), x)
    return x


def run_layer(ctx, name: str, W: Dict[str, torch.Tensor], state, batch, meta: dict) -> torch.Tensor:
    """One layer of the stack on a step batch: the residual rows in, the residual rows out (fp32);
    ``final.norm`` keeps the rows whose logits are wanted, ``head`` returns their logits."""
    cfg, ops = ctx.cfg, ctx.ops
    kind = layer_kind(name)
    if kind == "embed":
        out, ctx.embed_out = ctx.embed_out, None
        return ops.embed_rows(meta["ids"], W["embed"], out=out, scale=cfg.embedding_scale)
    if kind == "decoder":
        return run_block(ctx, W, state, meta, name)
    if kind == "norm":
        return ops.dyt_norm(state, W["norm"], W["alpha"], ctx.compute_dtype, row_idx=meta["want_idx"])
    return ops.matmul_nt(state, W["head"])


def layer_flops(cfg, name: str, rows: int, ctx_keys: float = 0.0) -> float:
    """Approximate forward FLOPs of decoder layer ``name`` on ``rows`` tokens (matrix products; the
    attention's score and value products over ``ctx_keys`` visible keys per row on average)."""
    L, D = cfg.layer(name), cfg.width
    m = L.mixer
    qs, ks, vs = _cols(m)
    H = m["heads"]
    keys = min(ctx_keys, float(_window(m) or NO_WINDOW))
    f = 2.0 * rows * D * (qs + ks + vs + H + H * m["vdim"]) + 2.0 * rows * keys * H * (m["dim"] + m["vdim"])
    if L.mlp is not None:
        r, fs = L.mlp["router"], _shared_ff(L.mlp)
        f += 2.0 * rows * D * (r["experts"] + 3 * r["top"] * L.mlp["expert"]["ff"] + 3 * fs + (1 if fs else 0))
    return f
