"""A plain, slow Gizezen forward pass in float64, one function per mechanism, written from the
design's equations.  It shares no code with the framework: the tests compare the framework's
kernels, caches and scheduler against it.

Notation: a sequence is a [T, D] matrix of rows x_t, t = 0 .. T-1 its positions; every function
takes the whole sequence and returns the whole output, recomputing everything from t = 0.
"""
import math

import torch

F = torch.float64


def dyt(x, w, b, alpha):
    """Dynamic Tanh: tanh(alpha x) w + b, elementwise (no statistics of the row)."""
    return torch.tanh(alpha * x) * w + b


def unit_rms(x, eps):
    """The last axis divided by sqrt(mean(x^2) + eps); no weight."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def short_conv(u, w):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j) per channel; rows before the start are zeros."""
    T, C = u.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F)
    for t in range(T):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] += w[:, j] * u[s]
    return out


def rot_freqs(rot):
    """f_i = base^(-2i / dims), then the wavelength-dependent rescaling: long waves (longer than
    original / low) slowed by ``factor``, short ones (shorter than original / high) kept, the band
    between blended linearly in original / wavelength."""
    dims, base = int(rot["dims"]), float(rot["base"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wl = 2 * math.pi / f
            if wl < orig / high:
                pass
            elif wl > orig / low:
                f = f / factor
            else:
                s = (orig / wl - low) / (high - low)
                f = (1 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, rot):
    """x: [T, heads, d].  Entries (2i, 2i + 1), i < dims / 2, of each head turn by the angle t f_i; the rest stay."""
    T = x.shape[0]
    out = x.clone()
    pos = torch.arange(T, dtype=F)
    for i, f in enumerate(rot_freqs(rot)):
        a = pos * f
        c, s = torch.cos(a)[:, None], torch.sin(a)[:, None]
        u, v = x[:, :, 2 * i], x[:, :, 2 * i + 1]
        out[:, :, 2 * i] = u * c - v * s
        out[:, :, 2 * i + 1] = v * c + u * s
    return out


def sees(i, j, size):
    return 0 <= i - j < size


def keys_values(h, m, W, eps):
    """What an attention layer caches: keys after convolution, rotation and unit norm; values after convolution."""
    T = h.shape[0]
    G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
    k = short_conv(h @ W["k"].T, W["k.conv"]).reshape(T, G, d)
    v = short_conv(h @ W["v"].T, W["v.conv"]).reshape(T, G, dv)
    return unit_rms(rotate(k, m["rot"]), eps), v


def sink_softmax(s):
    """p_j = exp(s_j) / (1 + sum_j exp(s_j)): a softmax with a silent extra entry of score 0."""
    mx = torch.clamp(s.max(), min=0.0)
    e = torch.exp(s - mx)
    return e / (torch.exp(-mx) + e.sum())


def attention(h, m, W, eps, shared=None):
    """``shared`` = (k, v) of the layer this one reads its keys and values from."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv(h @ W["q"].T, W["q.conv"]).reshape(T, H, d)
    q = unit_rms(rotate(q, m["rot"]), eps)
    k, v = shared if shared is not None else keys_values(h, m, W, eps)
    gate = torch.sigmoid(h @ W["g"].T)                        # [T, H]
    size = int(m["mask"]["size"])
    out = torch.zeros(T, H, dv, dtype=F)
    for i in range(T):
        js = [j for j in range(T) if sees(i, j, size)]
        for hh in range(H):
            g = hh // (H // G)
            s = (k[js, g] @ q[i, hh]) * m["scale"]
            p = sink_softmax(s)
            out[i, hh] = (p[:, None] * v[js, g]).sum(0) * gate[i, hh]
    return out.reshape(T, H * dv) @ W["o"].T


def route(z, top):
    """The ``top`` largest logits of each row and the softmax over just those."""
    vals, ids = torch.sort(z, dim=-1, descending=True, stable=True)
    return ids[:, :top], torch.softmax(vals[:, :top], -1)


def expert(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def moe(h, mlp, W):
    T = h.shape[0]
    ids, wts = route(h @ W["router"].T, int(mlp["router"]["top"]))
    out = torch.zeros(T, h.shape[1], dtype=F)
    for t in range(T):
        for e, w in zip(ids[t].tolist(), wts[t]):
            out[t] += w * expert(h[t:t + 1], W, f"e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W["shared.sg"].T) * expert(h, W, "shared.")
    return out


def sub(sd, prefix):
    return {k[len(prefix):]: v.to(F) for k, v in sd.items() if k.startswith(prefix)}


def norm_of(sd, name, x):
    return dyt(x, sd[name].to(F), sd[name + ".b"].to(F), sd[name + ".alpha"].to(F))


def forward(cfg, sd, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; ``layers_out``: a list that receives the residual stream after every layer."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x = sd["embed"].to(F)[torch.tensor(tokens)] * float(cfg["embedding"]["scale"])
    cached = {}
    for i, l in enumerate(cfg["layers"]):
        p, m = f"l{i}.", l["mixer"]
        W = sub(sd, p + "mix.")
        h = norm_of(sd, p + "norm1", x)
        if m.get("kv_from") is None:
            cached[i] = keys_values(h, m, W, eps)
            kv = cached[i]
        else:
            kv = cached[int(m["kv_from"])]
        x = x + mult * attention(h, m, W, eps, kv)
        if l.get("mlp") is not None:
            x = x + mult * moe(norm_of(sd, p + "norm2", x), l["mlp"], sub(sd, p + "mlp."))
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_of(sd, "final.norm", x) @ sd["head"].to(F).T
