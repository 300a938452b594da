"""A plain, slow Lopilix forward pass in float64, one function per mechanism, written from the
design's equations.  It shares no code with the framework: the tests compare the framework's
kernels, caches and scheduler against it.

Notation: a sequence is a [T, D] matrix of rows x_t, t = 0 .. T-1 its positions; every function
takes the whole sequence and returns the whole output, recomputing everything from t = 0.  ``sd``
maps tensor names to float64 tensors, ``cfg`` is config.json's content.
"""
import math

import torch

F = torch.float64


def rms(x, eps, w=None):
    """The last axis divided by sqrt(mean(x^2) + eps), times w when given."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def silu(z):
    return z * torch.sigmoid(z)


def gelu_erf(z):
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def rot_freqs(rot):
    """-> (frequencies f_i, i < dims / 2; the factor on every cosine and sine).  Without ``scaling``:
    f_i = base^(-2i / dims) and 1.  With it, by how many turns entry i makes over ``original``
    positions: entries below ``lo`` keep their frequency, entries above ``hi`` are slowed by
    ``factor``, a linear ramp between; lo / hi are the entry numbers whose turn counts are ``fast`` and
    ``slow``."""
    dims, base = int(rot["dims"]), float(rot["base"])
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, orig = float(sc["factor"]), float(sc["original"])

    def entry(turns):
        return dims * math.log(orig / (2 * math.pi * turns)) / (2 * math.log(base))

    lo = max(math.floor(entry(float(sc["fast"]))), 0)
    hi = min(math.ceil(entry(float(sc["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * ramp + fi * (1 - ramp))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x, rot, layout):
    """x: [T, heads, n].  Of each head's first ``dims`` entries, pairs (2i, 2i + 1) (``pairs``) or
    (i, i + dims / 2) (``half``) turn by the angle t f_i; the rest stay."""
    T = x.shape[0]
    dims = int(rot["dims"])
    freqs, amp = rot_freqs(rot)
    out = x.clone()
    pos = torch.arange(T, dtype=F)
    for i, f in enumerate(freqs):
        a, b = (2 * i, 2 * i + 1) if layout == "pairs" else (i, i + dims // 2)
        ang = pos * f
        c, s = (amp * torch.cos(ang))[:, None], (amp * torch.sin(ang))[:, None]
        u, v = x[:, :, a], x[:, :, b]
        out[:, :, a] = u * c - v * s
        out[:, :, b] = v * c + u * s
    return out


def causal_softmax_attention(q, k, v, scale):
    """q: [T, d], k: [T, d], v: [T, dv] of one head; row i sees keys j <= i."""
    T = q.shape[0]
    out = torch.zeros(T, v.shape[1], dtype=F)
    for i in range(T):
        s = (k[:i + 1] @ q[i]) * scale
        p = torch.softmax(s, 0)
        out[i] = p @ v[:i + 1]
    return out


def diff_lambda(sd, x, diff):
    return math.exp(float((sd[x + "lq1"] * sd[x + "lk1"]).sum())) - math.exp(float((sd[x + "lq2"] * sd[x + "lk2"]).sum())) + diff


def diff_attention(sd, x, m, h, eps):
    """Differential attention: every head holds two score maps over the same values; the second map's
    output is subtracted lambda times, the difference divided by its root mean square and scaled."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    diff = float(m["diff"])
    q = (h @ sd[x + "q"].T).reshape(T, H * 2, d)
    k = (h @ sd[x + "k"].T).reshape(T, G * 2, d)
    v = (h @ sd[x + "v"].T).reshape(T, G, dv)
    q, k = rms(q, eps, sd[x + "q.norm"]), rms(k, eps, sd[x + "k.norm"])
    if m.get("rot"):
        q, k = rotate(q, m["rot"], "pairs"), rotate(k, m["rot"], "pairs")
    lam = diff_lambda(sd, x, diff)
    out = torch.zeros(T, H, dv, dtype=F)
    for hh in range(H):
        g = hh // (H // G)
        a1 = causal_softmax_attention(q[:, 2 * hh], k[:, 2 * g], v[:, g], float(m["scale"]))
        a2 = causal_softmax_attention(q[:, 2 * hh + 1], k[:, 2 * g + 1], v[:, g], float(m["scale"]))
        out[:, hh] = rms(a1 - lam * a2, eps) * (1.0 - diff)
    return out.reshape(T, H * dv) @ sd[x + "o"].T


def hgrn2(sd, x, m, h, eps):
    """Gated linear recurrence: the forget gate f decays the state's rows and 1 - f is what is written."""
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ sd[x + "q"].T).reshape(T, H, d)
    low = sd[x + "lower"]
    f = (low + (1 - low) * torch.sigmoid(h @ sd[x + "f"].T + sd[x + "f.b"])).reshape(T, H, d)
    v = (h @ sd[x + "v"].T).reshape(T, H, dv)
    S = torch.zeros(H, d, dv, dtype=F)
    out = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        S = f[t][:, :, None] * S + (1 - f[t])[:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hkv,hk->hv", S, q[t])
    return rms(out, eps, sd[x + "norm"]).reshape(T, H * dv) @ sd[x + "o"].T


def latent_attention(sd, x, m, h, eps):
    """Keys and values are linear maps of one normed latent row per token, plus one rotated key part
    that all heads share; the heads' outputs are gated by a sigmoid of the input."""
    T = h.shape[0]
    H, d, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ sd[x + "q"].T).reshape(T, H, d + dr)
    ckr = h @ sd[x + "dkv"].T
    c = rms(ckr[:, :r], eps, sd[x + "dkv.norm"])
    kr = ckr[:, r:].reshape(T, 1, dr)
    qn, qr = q[:, :, :d], q[:, :, d:]
    if m.get("rot"):
        qr, kr = rotate(qr, m["rot"], "half"), rotate(kr, m["rot"], "half")
    kn = (c @ sd[x + "uk"].T).reshape(T, H, d)
    v = (c @ sd[x + "uv"].T).reshape(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F)
    for hh in range(H):
        out[:, hh] = causal_softmax_attention(torch.cat([qn[:, hh], qr[:, hh]], 1), torch.cat([kn[:, hh], kr[:, 0]], 1),
                                              v[:, hh], float(m["scale"]))
    o = out.reshape(T, H * dv) * torch.sigmoid(h @ sd[x + "g"].T)
    return o @ sd[x + "o"].T


def dense_ff(sd, y, h):
    g = h @ sd[y + "gate"].T + sd[y + "gate.b"]
    u = h @ sd[y + "up"].T + sd[y + "up.b"]
    return (silu(g) * u) @ sd[y + "down"].T + sd[y + "down.b"]


def route(z, r):
    """z: router logits of one token [E] -> [(expert, weight)].  Scores are sigmoids; a group of
    neighbouring experts is worth the sum of its two best scores; only the best groups' experts compete."""
    E, top = int(r["experts"]), int(r["top"])
    s = torch.sigmoid(z)
    allowed = list(range(E))
    gr = r.get("groups")
    if gr:
        n, keep = int(gr["count"]), int(gr["keep"])
        size = E // n
        worth = []
        for g in range(n):
            best = sorted((float(s[e]) for e in range(g * size, (g + 1) * size)), reverse=True)
            worth.append(sum(best[:2]))
        kept = sorted(range(n), key=lambda g: (-worth[g], g))[:keep]
        allowed = [e for e in range(E) if e // size in kept]
    chosen = sorted(allowed, key=lambda e: (-float(s[e]), e))[:top]
    tot = sum(float(s[e]) for e in chosen) + 1e-20
    return [(e, float(s[e]) / tot * float(r.get("scale", 1.0))) for e in chosen]


def moe_ff(sd, y, mlp, h):
    T = h.shape[0]
    z = h @ sd[y + "router"].T
    out = torch.zeros(T, sd[y + "e0.down"].shape[0], dtype=F)
    for t in range(T):
        for e, w in route(z[t], mlp["router"]):
            out[t] += w * (gelu_erf(h[t] @ sd[f"{y}e{e}.up"].T) @ sd[f"{y}e{e}.down"].T)
    return out


def sublayer(sd, cfg, i, which, h):
    L = cfg["layers"][i]
    eps = float(cfg["norm"]["eps"])
    if which == 1:
        fn = {"attention": diff_attention, "hgrn2": hgrn2, "latent_attention": latent_attention}[L["type"]]
        return fn(sd, f"l{i}.mix.", L["mixer"], h, eps)
    if L["mlp"]["kind"] == "dense":
        return dense_ff(sd, f"l{i}.mlp.", h)
    return moe_ff(sd, f"l{i}.mlp.", L["mlp"], h)


def layer(sd, cfg, i, xs):
    """xs: [S, T, D], the residual streams -> the streams after layer i.  Sublayer q reads
    u = sum_s in[s] xs[s]; its output, gated by sigmoid(W norm(u) + b), joins stream t times out[t]
    while the streams are mixed by mix[from, to]."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    for which in (1, 2):
        if which == 2 and cfg["layers"][i].get("mlp") is None:
            break
        p = f"l{i}."
        cin, cout, mix = sd[f"{p}hc{which}.in"], sd[f"{p}hc{which}.out"], sd[f"{p}hc{which}.mix"]
        u = torch.einsum("s,std->td", cin, xs)
        h = rms(u, eps, sd[f"{p}norm{which}"])
        y = sublayer(sd, cfg, i, which, h)
        y = y * torch.sigmoid(h @ sd[f"{p}rg{which}"].T + sd[f"{p}rg{which}.b"])
        xs = torch.einsum("sr,std->rtd", mix, xs) + mult * cout[:, None, None] * y[None]
    return xs


def layer_order(cfg):
    """Layer numbers in the order they run: layers start .. stop - 1 repeat ``times`` times in a row."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    a, b, k = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return list(range(a)) + list(range(a, b)) * k + list(range(b, n))


def forward(sd, cfg, tokens, trace=None):
    """tokens: list of ids -> logits [T, vocab].  ``trace``: a list that receives the summed streams
    after every layer run."""
    T = len(tokens)
    x = sd["embed"][torch.tensor(tokens)] + sd["pos"][:T]
    xs = x[None].repeat(int(cfg.get("streams", 1)), 1, 1)
    for i in layer_order(cfg):
        xs = layer(sd, cfg, i, xs)
        if trace is not None:
            trace.append(xs.sum(0))
    h = rms(xs.sum(0), float(cfg["norm"]["eps"]), sd["final.norm"])
    return (h @ sd["embed"].T) * float(cfg["logit_scale"])
