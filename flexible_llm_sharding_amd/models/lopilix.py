"""Lopilix layer execution on packed weight images and packed step batches.

The activation between layers is ``streams`` residual streams per row, side by side ([T, streams * D]
fp32; all start as the embedding row plus a learned position vector).  Sublayer q of a layer (1: the
mixer, 2: the feed-forward) is

    h = rms_norm(sum_s in_q[s] x_s);   y = sublayer(h) * sigmoid(W_rg h + b_rg)
    x_t <- sum_s mix_q[s, t] x_s + m * out_q[t] * y          (all streams at once, m = ``residual_mult``)

Mixers:

* ``attention`` -- differential attention.  q and k hold two score maps per head, each RMS-normed per
  head with a shared weight and rotated in pairs (2i, 2i + 1) over the first ``rot.dims`` entries; both
  maps are softmax attentions over the same values, o = a1 - lambda a2 with one lambda per layer
  (exp(lq1 . lk1) - exp(lq2 . lk2) + diff), o divided by its root mean square per head, times (1 - diff).
  The image stores q and k map by map (all heads of map 1, then all of map 2), so the two maps are
  2 H query heads over 2 G key heads of an ordinary grouped-query attention whose value head is the key
  head modulo G;
* ``hgrn2`` -- per head a state S [dim, vdim]: S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T silu(q_t)
  with the forget gate f = lower + (1 - lower) sigmoid(W_f h + b); o RMS-normed per head;
* ``latent_attention`` -- softmax attention whose keys and values are linear maps of one cached latent
  row c_j (RMS-normed) plus a rotated key part shared by all heads (pairs (i, i + dims / 2), frequencies
  rescaled by how often a pair turns over the original context, cosines and sines amplified); the
  heads' outputs are gated by sigmoid(W_g h).  Steps that continue a sequence fold W_uk into the query
  and W_uv behind the attention, which then runs with one key/value head over the latent rows; whole
  prompts make per-head keys and values from the step's rows.

Feed-forwards: W_down(silu(W_gate h + b) * (W_up h + b)) + b, or a mixture of experts
W_down gelu(W_up h) chosen by sigmoid scores among the best groups of experts, weighted by
score / sum of the chosen * ``router.scale``.  The first product of every sublayer also makes the
residual gate's logits (its rows are stacked under the projections).  Each mechanism is an op of the
backend (``ops/hip_seq.py``: the kernels of ``csrc/kernels/seq``; ``ops/torch_seq.py`` on the CPU)
with its constants as arguments; this file only strings them together.  Keys, values, latent rows and
recurrent states live in :class:`~..runtime.seq_state.SequenceStateCache`, one set per pass of a looped
layer.
"""
from __future__ import annotations

from typing import Dict, List

import torch

from .kagolix import HybridContext  # noqa: F401  (the context the engine builds for every hybrid family)
from .layout import LayerLayout, Placement, layer_image, layer_kind, spec_layout, spec_placements

F32 = "f32"
NO_WINDOW = 1 << 30                # every earlier key is visible


def _rot(m: dict):
    """(dims, base, scaling) of the rotation for ``head_norm_rope``, or None."""
    r = m.get("rot")
    if not r or int(r["dims"]) < 2:
        return None
    s = r.get("scaling")
    sc = ("turns", float(s["factor"]), float(s["original"]), float(s["fast"]), float(s["slow"])) if s else None
    return int(r["dims"]), float(r["base"]), sc


def _mixer_cols(L) -> Dict[str, tuple]:
    """Column ranges (start, width) of a mixer's stacked input projection (without the residual gate)."""
    m = L.mixer
    if L.type == "attention":
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        widths = [("q", 2 * H * d), ("k", 2 * G * d), ("v", G * dv)]
    elif L.type == "hgrn2":
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        widths = [("q", H * d), ("f", H * d), ("v", H * dv)]
    else:
        H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        widths = [("q", H * (d + dr)), ("dkv", r + dr), ("g", H * dv)]
    out, at = {}, 0
    for n, w in widths:
        out[n] = (at, int(w))
        at += int(w)
    out["all"] = (0, at)
    return out


def _hc_specs(cfg, slot: str, tensor: str):
    s = cfg.streams
    if not cfg.hyper:
        return []
    return [(slot, (2 * s + s * s,), F32, [(tensor + ".in", 0, (s,)), (tensor + ".out", s, (s,)), (tensor + ".mix", 2 * s, (s, s))])]


def _specs(cfg, name: str):
    """[(slot, shape, dtype tag, [(checkpoint tensor, element offset in the slot, shape[, options])])]."""
    D, V = cfg.width, cfg.vocab
    kind = layer_kind(name)
    if kind == "embed":
        return [("embed", (V, D), None, [("embed", 0, (V, D))]),
                ("pos", (cfg.max_positions, D), None, [("pos", 0, (cfg.max_positions, D))])]
    if kind == "head":
        return [("head", (V, D), None, [("embed", 0, (V, D))])]        # the logits come from the embedding table
    if kind == "norm":
        return [("norm", (D,), F32, [("final.norm", 0, (D,))])]
    name = layer_image(name)
    L, p = cfg.layer(name), name + "."
    m, x = L.mixer, name + ".mix."
    c = _mixer_cols(L)
    n_in = c["all"][1]
    gate = D if cfg.gated else 0
    out = [("norm1", (D,), F32, [(p + "norm1", 0, (D,))])] + _hc_specs(cfg, "hc1", p + "hc1")
    rg = [(p + "rg1", n_in * D, (D, D))] if gate else []
    rgb = [(p + "rg1.b", n_in, (D,))] if gate else []
    if L.type == "attention":
        H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        # q and k: the checkpoint lays a head's two maps side by side; the image holds map 1 of all heads, then map 2
        by_map = lambda n: {"view": (n, 2, d, D), "perm": (1, 0, 2, 3)}
        out += [("win", (n_in + gate, D), None,
                 [(x + "q", 0, (2 * H * d, D), by_map(H)), (x + "k", c["k"][0] * D, (2 * G * d, D), by_map(G)),
                  (x + "v", c["v"][0] * D, (G * dv, D))] + rg),
                ("qn", (d,), F32, [(x + "q.norm", 0, (d,))]), ("kn", (d,), F32, [(x + "k.norm", 0, (d,))]),
                ("lam", (4, d), F32, [(x + "lq1", 0, (d,)), (x + "lk1", d, (d,)), (x + "lq2", 2 * d, (d,)), (x + "lk2", 3 * d, (d,))]),
                ("wo", (D, H * dv), None, [(x + "o", 0, (D, H * dv))])]
        if gate:
            out.append(("bin", (n_in + gate,), F32, rgb))
    elif L.type == "hgrn2":
        H, d, dv = m["heads"], m["dim"], m["vdim"]
        out += [("win", (n_in + gate, D), None,
                 [(x + "q", 0, (H * d, D)), (x + "f", c["f"][0] * D, (H * d, D)), (x + "v", c["v"][0] * D, (H * dv, D))] + rg),
                ("bin", (n_in + gate,), F32, [(x + "f.b", c["f"][0], (H * d,))] + rgb),
                ("lower", (H * d,), F32, [(x + "lower", 0, (H * d,))]), ("mnorm", (dv,), F32, [(x + "norm", 0, (dv,))]),
                ("wo", (D, H * dv), None, [(x + "o", 0, (D, H * dv))])]
    else:
        H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
        out += [("win", (n_in + gate, D), None,
                 [(x + "q", 0, (H * (d + dr), D)), (x + "dkv", c["dkv"][0] * D, (r + dr, D)), (x + "g", c["g"][0] * D, (H * dv, D))] + rg),
                ("dkvn", (r,), F32, [(x + "dkv.norm", 0, (r,))]),
                # W_uk per head, transposed: the product that folds it into the queries reads it as [N = r, K = d]
                ("wukt", (H, r, d), None, [(x + "uk", 0, (H * d, r), {"view": (H, d, r), "perm": (0, 2, 1)})]),
                ("wuk", (H, d, r), None, [(x + "uk", 0, (H * d, r))]),
                ("wuv", (H, dv, r), None, [(x + "uv", 0, (H * dv, r))]),
                ("wo", (D, H * dv), None, [(x + "o", 0, (D, H * dv))])]
        if gate:
            out.append(("bin", (n_in + gate,), F32, rgb))
    if L.mlp is not None:
        y = p + "mlp."
        out += [("norm2", (D,), F32, [(p + "norm2", 0, (D,))])] + _hc_specs(cfg, "hc2", p + "hc2")
        if L.mlp["kind"] == "dense":
            ff = int(L.mlp["ff"])
            out += [("wgu", (2 * ff + gate, D), None,
                     [(y + "gate", 0, (ff, D)), (y + "up", ff * D, (ff, D))] + ([(p + "rg2", 2 * ff * D, (D, D))] if gate else [])),
                    ("bgu", (2 * ff + gate,), F32,
                     [(y + "gate.b", 0, (ff,)), (y + "up.b", ff, (ff,))] + ([(p + "rg2.b", 2 * ff, (D,))] if gate else [])),
                    ("wdown", (D, ff), None, [(y + "down", 0, (D, ff))]), ("bdown", (D,), F32, [(y + "down.b", 0, (D,))])]
        else:
            E, ff = int(L.mlp["router"]["experts"]), int(L.mlp["expert"]["ff"])
            out += [("wrr", (E + gate, D), None, [(y + "router", 0, (E, D))] + ([(p + "rg2", E * D, (D, D))] if gate else [])),
                    ("wup", (E, ff, D), None, [(f"{y}e{e}.up", e * ff * D, (ff, D)) for e in range(E)]),
                    ("wdown", (E, D, ff), None, [(f"{y}e{e}.down", e * D * ff, (D, ff)) for e in range(E)])]
            if gate:
                out.append(("brr", (E + gate,), F32, [(p + "rg2.b", E, (D,))]))
    return out


def layout(cfg, name: str, elem_size: int = 2) -> LayerLayout:
    return spec_layout(layer_kind(name), _specs(cfg, name), elem_size)


def placements(cfg, name: str, elem_size: int = 2) -> List[Placement]:
    return spec_placements(layout(cfg, name, elem_size), _specs(cfg, name), elem_size)


def state_spec(cfg) -> dict:
    """What a request keeps between steps, per pass of every layer: keys (both maps) and values of a
    differential attention, latent rows [c | rotated key part] of a latent attention, the fp32 state of an
    HGRN2 layer.  Nothing is ever behind a horizon: every earlier key stays visible."""
    paged, slots, horizons = {}, {}, []
    for name in cfg.layer_names():
        if layer_kind(name) != "decoder":
            continue
        L = cfg.layer(name)
        m = L.mixer
        if L.type == "attention":
            paged[name] = {"k": 2 * m["kv_heads"] * m["dim"], "v": m["kv_heads"] * m["vdim"]}
            horizons.append(("window", NO_WINDOW, 0))
        elif L.type == "latent_attention":
            paged[name] = {"ckr": int(m["kv_rank"]) + int(m["rot_dim"])}
            horizons.append(("window", NO_WINDOW, 0))
        else:
            slots[name] = {"state": (m["heads"], m["dim"], m["vdim"])}
    return {"paged": paged, "alias": {}, "slots": slots, "horizons": horizons}


# ------------------------------------------------------------------------------------ execution
def _gate_cols(cfg, z, n_in: int):
    return z[:, n_in:n_in + cfg.width] if cfg.gated else None


def _diff_attention(ctx, L, W, h, meta, name: str):
    ops, eps, cdt, m = ctx.ops, ctx.cfg.norm_eps, ctx.compute_dtype, L.mixer
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    c = _mixer_cols(L)
    z = ops.matmul_nt(h, W["win"], bias=W.get("bin"))                      # fp32 [T, q (by map) | k (by map) | v | gate]
    T = z.shape[0]
    kc, vc = ctx.cache.kv(name)
    rot = _rot(m)
    q = torch.empty(T, 2 * H * d, dtype=torch.float32, device=z.device)
    # per head and map: norm with the shared weight, rotation; q to fp32 rows, k and v into their pages
    if rot is None or rot[2] is None:
        ops.qkv_conv_rope_store(z, None, None, meta, 2 * H, 2 * G, d, dv, q, kc, vc, eps=eps, rot=rot, v_heads=G, q_norm=W["qn"],
                                k_norm=W["kn"])                              # (one pass)
    else:       # rescaled frequencies carry an amplitude on cosines and sines, which the per-head op applies
        ops.head_norm_rope(z, 2 * H, d, 0, d, q, 0, d, meta, w=W["qn"], eps=eps, rot=rot)
        ops.head_norm_rope(z, 2 * G, d, c["k"][0], d, kc.view(-1, kc.shape[-1]), 0, d, meta, w=W["kn"], eps=eps, rot=rot,
                           row_map=meta["kv_slot"])
        ops.head_norm_rope(z, G, dv, c["v"][0], dv, vc.view(-1, vc.shape[-1]), 0, dv, meta, row_map=meta["kv_slot"])
    # the two maps as 2 H heads over 2 G key heads; both maps of a key head read the same value head
    a = torch.empty(T, 2 * H * dv, dtype=torch.float32, device=z.device)
    ops.attn_paged(q, kc, vc, meta, 2 * H, 2 * G, d, dv, scale=float(m["scale"]), softcap=0.0, r1=None, r2=None, chunk=0,
                   page_size=ctx.cache.page_size, out_dtype=cdt, out=a, v_heads=G)
    o = ops.diff_combine(a, W["lam"], float(m["diff"]), H, dv, eps, cdt)
    return ops.matmul_nt(o, W["wo"]), _gate_cols(ctx.cfg, z, c["all"][1])


def _hgrn2(ctx, L, W, h, meta, name: str):
    ops, m = ctx.ops, L.mixer
    c = _mixer_cols(L)
    col = lambda z, n: z[:, c[n][0]:c[n][0] + c[n][1]]
    z = ops.matmul_nt(h, W["win"], bias=W["bin"])                          # fp32 [T, q | f + b | v | gate]
    st = ctx.cache.recurrent(name)["state"]
    o = ops.hgrn2_scan(col(z, "q"), col(z, "f"), col(z, "v"), None, W["lower"], W["mnorm"], st, meta, m["heads"], m["dim"],
                       m["vdim"], ctx.cfg.norm_eps, ctx.compute_dtype)
    return ops.matmul_nt(o, W["wo"]), _gate_cols(ctx.cfg, z, c["all"][1])


def _latent_attention(ctx, L, W, h, meta, name: str):
    ops, eps, cdt, m = ctx.ops, ctx.cfg.norm_eps, ctx.compute_dtype, L.mixer
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    c = _mixer_cols(L)
    rot = _rot(m)
    scale = float(m["scale"])
    pool = ctx.cache.pools(name)["ckr"]                                   # [pages, page, c | kr]
    z = ops.matmul_nt(h, W["win"], bias=W.get("bin"))                      # fp32 [T, q | c | kr | g | gate]
    T, k0 = z.shape[0], c["dkv"][0]
    q = z[:, :H * (d + dr)]
    rows = pool.view(-1, r + dr)
    ops.head_norm_rope(z, 1, r, k0, 0, rows, 0, 0, meta, w=W["dkvn"], eps=eps, row_map=meta["kv_slot"])
    ops.head_norm_rope(z, 1, dr, k0 + r, 0, rows, r, 0, meta, rot=rot, row_map=meta["kv_slot"], half=True)
    g = z[:, c["g"][0]:c["g"][0] + H * dv]
    local = meta.get("local_table")
    if local is not None and ops.unfolded_attention_ok(d + dr, dv, cdt):
        # whole prompts (every request of the step starts at position 0, so all keys are this step's rows):
        # keys and values are made per head from the rows as cached, [W_uk,h c | kr] and W_uv,h c
        ckr = ops.gather_rows(rows, meta["kv_slot"])                      # [T, c | kr]
        kf = torch.empty(T, H * (d + dr), dtype=cdt, device=z.device)
        ops.head_matmul_nt(ckr, W["wuk"], H, 0, kf, d + dr)
        ops.head_norm_rope(ckr, H, dr, r, 0, kf, d, d + dr, meta)         # the one rotated part beside every head's keys
        vf = ops.matmul_nt(ckr[:, :r], W["wuv"].view(H * dv, r), out_dtype=cdt)
        ops.head_norm_rope(q, H, dr, d, d + dr, q, d, d + dr, meta, rot=rot, half=True)        # (in place)
        a = torch.empty(T, H * dv, dtype=torch.float32, device=z.device)
        ops.attn_paged(q, kf.view(T, 1, -1), vf.view(T, 1, -1), dict(meta, page_table=local), H, H, d + dr, dv, scale=scale,
                       softcap=0.0, r1=None, r2=None, chunk=0, page_size=1, out_dtype=cdt, out=a)
        o = ops.sigmoid_gate(a, g, cdt)
    else:
        # decoding, portions: the query each head asks the latent rows with is [W_uk,h^T q_unrotated | q_rotated]
        qa = torch.empty(T, H * (r + dr), dtype=torch.float32, device=z.device)
        ops.head_matmul_nt(q, W["wukt"], H, d + dr, qa, r + dr)
        ops.head_norm_rope(q, H, dr, d, d + dr, qa, r, r + dr, meta, rot=rot, half=True)
        a = ops.attn_paged(qa, pool, pool, meta, H, 1, r + dr, r, scale=scale, softcap=0.0, r1=None, r2=None, chunk=0,
                           page_size=ctx.cache.page_size, out_dtype=cdt)
        ov = torch.empty(T, H * dv, dtype=torch.float32, device=z.device)
        ops.head_matmul_nt(a, W["wuv"], H, r, ov, dv)                     # each head's weighted latent -> its values
        o = ops.sigmoid_gate(ov, g, cdt)
    return ops.matmul_nt(o, W["wo"]), _gate_cols(ctx.cfg, z, c["all"][1])


def _dense(ctx, mlp: dict, W, h):
    ops, cdt = ctx.ops, ctx.compute_dtype
    ff = int(mlp["ff"])
    z = ops.matmul_nt(h, W["wgu"], bias=W["bgu"])                          # fp32 [T, gate | up | residual gate]
    y = ops.matmul_nt(ops.gate_mul(z[:, :2 * ff], cdt, act="silu"), W["wdown"], bias=W["bdown"])
    return y, _gate_cols(ctx.cfg, z, 2 * ff)


def _moe(ctx, mlp: dict, W, h):
    ops, cdt = ctx.ops, ctx.compute_dtype
    r = mlp["router"]
    E = int(r["experts"])
    g = r.get("groups") or {}
    z = ops.matmul_nt(h, W["wrr"], bias=W.get("brr"))                      # fp32 [T, router logits | residual gate]
    route = ops.moe_route_grouped(z[:, :E], int(r["top"]), int(g.get("count", 0)), int(g.get("keep", 0)), float(r.get("scale", 1.0)))
    hp = ops.gather_rows(h, route.rows)                                   # rows sorted by expert
    up = ops.grouped_matmul_nt(hp, W["wup"], route.offs)                  # fp32 [T top, ff]
    yo = ops.grouped_matmul_nt(ops.unary(up, "gelu", cdt), W["wdown"], route.offs)
    return ops.moe_weighted_sum(yo, route), _gate_cols(ctx.cfg, z, E)


_MIXERS = {"attention": _diff_attention, "hgrn2": _hgrn2, "latent_attention": _latent_attention}


def run_block(ctx, W, xs: torch.Tensor, meta: dict, name: str) -> torch.Tensor:
    cfg, ops, cdt = ctx.cfg, ctx.ops, ctx.compute_dtype
    L = cfg.layer(name)
    S, eps, mult = cfg.streams, cfg.norm_eps, cfg.residual_mult
    hc1, hc2 = W.get("hc1"), W.get("hc2")
    h = ops.streams_norm(xs, hc1, W["norm1"], eps, cdt, S)
    y, gate = _MIXERS[L.type](ctx, L, W, h, meta, name)
    if L.mlp is None:
        return ops.streams_update_(xs, y, gate, hc1, mult, S)
    # (the streams' update and the feed-forward's norm read and write the streams once)
    h = ops.streams_update_norm_(xs, y, gate, hc1, mult, S, hc2, W["norm2"], eps, cdt)
    y, gate = (_dense if L.mlp["kind"] == "dense" else _moe)(ctx, L.mlp, W, h)
    return ops.streams_update_(xs, y, gate, hc2, mult, S)


def run_layer(ctx, name: str, W: Dict[str, torch.Tensor], state, batch, meta: dict) -> torch.Tensor:
    """One layer of the stack on a step batch: the residual streams in, the residual streams out (fp32);
    ``final.norm`` sums the streams of the rows whose logits are wanted and norms them, ``head`` returns
    their logits."""
    cfg, ops = ctx.cfg, ctx.ops
    kind = layer_kind(name)
    if kind == "embed":
        out, ctx.embed_out = ctx.embed_out, None
        return ops.embed_rows(meta["ids"], W["embed"], out=out, pos_table=W["pos"], tok_pos=meta["tok_pos"], copies=cfg.streams)
    if kind == "decoder":
        return run_block(ctx, W, state, meta, name)
    if kind == "norm":
        return ops.streams_norm(state, None, W["norm"], cfg.norm_eps, ctx.compute_dtype, cfg.streams, row_idx=meta["want_idx"])
    z = ops.matmul_nt(state, W["head"])
    return ops.scale_(z, cfg.logit_scale) if cfg.logit_scale != 1.0 else z


def layer_flops(cfg, name: str, rows: int, ctx_keys: float = 0.0) -> float:
    """Approximate forward FLOPs of decoder layer ``name`` on ``rows`` tokens (matrix products; the
    attention's score and value products over ``ctx_keys`` visible keys per row on average)."""
    L, D = cfg.layer(name), cfg.width
    m = L.mixer
    gate = D if cfg.gated else 0
    n_in = _mixer_cols(L)["all"][1]
    H, dv = m["heads"], m["vdim"]
    f = 2.0 * rows * D * (n_in + gate + H * dv)
    if L.type == "attention":
        f += 4.0 * rows * ctx_keys * H * (m["dim"] + dv)
    elif L.type == "hgrn2":
        f += 6.0 * rows * H * m["dim"] * dv
    else:
        r, dr = m["kv_rank"], m["rot_dim"]
        f += 2.0 * rows * (H * m["dim"] * r + H * r * dv) + 2.0 * rows * ctx_keys * H * (2 * r + dr)
    if L.mlp is not None:
        if L.mlp["kind"] == "dense":
            f += 2.0 * rows * D * (3 * int(L.mlp["ff"]) + gate)
        else:
            f += 2.0 * rows * D * (L.mlp["router"]["experts"] + gate + 2 * L.mlp["router"]["top"] * L.mlp["expert"]["ff"])
    return f
