"""Plain-PyTorch ops of the stateful (hybrid) models: the CPU path and the layer-by-layer check of
the HIP kernels in ``csrc/kernels/seq``.  Same signatures as ``hip_seq.HipSeqOps``.

Norms, scores, softmax, gates and recurrences run in fp32 whatever the GEMM element type; a GEMM
takes operands of the weight's type and returns its fp32 accumulator.
"""
from __future__ import annotations

import math
from dataclasses import dataclass

import torch
import torch.nn.functional as F


@dataclass
class SeqRoute:
    """Routing of one mixture-of-experts call: per (token, choice) the expert and its weight; rows
    sorted by expert (``rows``: sorted row -> token, ``dest``: (token, choice) -> sorted row) and each
    expert's range of sorted rows (``offs``)."""
    ids: torch.Tensor
    w: torch.Tensor
    offs: torch.Tensor
    rows: torch.Tensor
    dest: torch.Tensor
    top: int


class TorchSeqOps:
    # ----------------------------------------------------------------- rows
    def embed_rows(self, ids, table, out=None, scale=1.0, pos_table=None, tok_pos=None, copies=1):
        """out[t] = table[ids[t]] * scale (+ pos_table[tok_pos[t]], a learned position vector), written
        ``copies`` times side by side (the start of that many residual streams)."""
        e = table.index_select(0, ids.long()).float()
        if scale != 1.0:
            e = e * scale
        if pos_table is not None:
            e = e + pos_table.index_select(0, tok_pos.long()).float()
        if copies > 1:
            e = e.repeat(1, copies)
        if out is not None:
            out.copy_(e)
            return out
        return e

    def group_rmsnorm(self, x, w, groups, eps, out_dtype, row_idx=None, w_offset=0.0):
        """``w_offset``: added to the weight (1.0 for weights stored around zero)."""
        if row_idx is not None:
            x = x.index_select(0, row_idx.long())
        T, D = x.shape
        p = x.float().reshape(T, groups, D // groups)
        p = p * torch.rsqrt(p.pow(2).mean(-1, keepdim=True) + eps)
        return (p.reshape(T, D) * (w.float() + w_offset)).to(out_dtype)

    def add_group_rmsnorm_(self, x, y, w, groups, eps, w_offset=0.0):
        x.add_(self.group_rmsnorm(y, w, groups, eps, torch.float32, w_offset=w_offset))
        return x

    def dyt_norm(self, x, wb, alpha, out_dtype, row_idx=None):
        """Dynamic Tanh: tanh(alpha x) w + b elementwise, no statistics of the row; ``wb`` = [w; b] ([2, D]),
        ``alpha`` a one-element tensor."""
        if row_idx is not None:
            x = x.index_select(0, row_idx.long())
        return (torch.tanh(alpha.float() * x.float()) * wb[0].float() + wb[1].float()).to(out_dtype)

    def add_scaled_(self, x, y, mult):
        """x += mult * y (the residual update of a sublayer whose output joins the stream scaled)."""
        x.add_(y.float(), alpha=float(mult))
        return x

    def add_scaled_dyt_norm_(self, x, y, mult, wb, alpha, out_dtype):
        """x += mult * y, and the Dynamic Tanh norm of the new x for the next sublayer, in one pass."""
        self.add_scaled_(x, y, mult)
        return self.dyt_norm(x, wb, alpha, out_dtype)

    def streams_norm(self, xs, coef, w, eps, out_dtype, streams, row_idx=None):
        """xs: [T, streams * D], the residual streams of a row side by side.  u = sum_s coef[s] xs_s
        (``coef`` None: the plain sum), then u / sqrt(mean(u^2) + eps) * w."""
        if row_idx is not None:
            xs = xs.index_select(0, row_idx.long())
        T = xs.shape[0]
        x3 = xs.float().reshape(T, streams, xs.shape[1] // streams)
        u = x3.sum(1) if coef is None else torch.einsum("s,tsd->td", coef.float()[:streams], x3)
        return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)

    def streams_update_(self, xs, y, gate, hc, mult, streams):
        """All streams at once from the old ones: xs_t <- sum_s mix[s, t] xs_s + mult * out[t] * y * sigmoid(gate).
        ``hc`` = [in (streams) | out (streams) | mix (streams x streams, [from, to])] fp32, None: one stream
        that keeps itself (a plain residual sum); ``gate`` [T, D] fp32 logits or None."""
        T = xs.shape[0]
        x3 = xs.reshape(T, streams, xs.shape[1] // streams)
        yy = y.float()
        if gate is not None:
            yy = yy * torch.sigmoid(gate.float())
        if hc is None:
            xs.add_(yy.repeat(1, streams), alpha=float(mult))
            return xs
        out, mix = hc[streams:2 * streams].float(), hc[2 * streams:].float().reshape(streams, streams)
        new = torch.einsum("sr,tsd->trd", mix, x3.float()) + float(mult) * out[None, :, None] * yy[:, None, :]
        xs.copy_(new.reshape(T, -1))
        return xs

    def streams_update_norm_(self, xs, y, gate, hc, mult, streams, coef, w, eps, out_dtype):
        """``streams_update_`` and the next sublayer's ``streams_norm`` of the new streams, in one pass."""
        self.streams_update_(xs, y, gate, hc, mult, streams)
        return self.streams_norm(xs, coef, w, eps, out_dtype, streams)

    def scale_(self, z, alpha):
        z.mul_(float(alpha))
        return z

    def sigmoid_gate(self, o, g, out_dtype):
        """o * sigmoid(g), element by element."""
        return (o.float() * torch.sigmoid(g.float())).to(out_dtype)

    def matmul_nt(self, a, w, bias=None, xielu=None, out_dtype=torch.float32):
        if a.dtype != w.dtype:
            a = a.to(w.dtype)
        y = (a @ w.t()).float() if w.dtype == torch.float32 else (a.float() @ w.float().t())
        if bias is not None:
            y = y + bias.float()
        if xielu is not None:
            return self.xielu(y, xielu, out_dtype)
        return y.to(out_dtype)

    def block_linear(self, u, w, b, blocks, cdt):
        """[T, blocks * bw] -> [T, G * bw]: column block g of the output is block g % blocks of
        u (rounded to ``cdt``) times w[g]^T, plus b."""
        T, Wd = u.shape
        G, bw, _ = w.shape
        ub = u.to(cdt).float().reshape(T, blocks, bw)
        ub = ub.repeat(1, G // blocks, 1)
        return torch.einsum("tgi,goi->tgo", ub, w.float()).reshape(T, G * bw) + b.float()

    def xielu(self, z, act, out_dtype):
        ap, an = F.softplus(act[0].float()), 0.5 + F.softplus(act[1].float())
        z = z.float()
        pos = ap * z * z + 0.5 * z
        neg = an * (torch.expm1(torch.clamp(z, max=0.0)) - z) + 0.5 * z
        return torch.where(z > 0, pos, neg).to(out_dtype)

    def gate_mul(self, gu, out_dtype, act="silu"):
        """act(gu[:, :ff]) * gu[:, ff:]; act: silu or gelu_tanh."""
        ff = gu.shape[1] // 2
        g, u = gu[:, :ff].float(), gu[:, ff:].float()
        if act == "silu":
            a = g * torch.sigmoid(g)
        elif act == "gelu_tanh":
            a = 0.5 * g * (1 + torch.tanh(math.sqrt(2 / math.pi) * (g + 0.044715 * g ** 3)))
        else:
            raise ValueError(act)
        return (a * u).to(out_dtype)

    def silu_mul(self, gu, out_dtype):
        return self.gate_mul(gu, out_dtype, "silu")

    def unary(self, z, kind, out_dtype):
        """tanh, or gelu: the exact form 0.5 z (1 + erf(z / sqrt 2))."""
        if kind == "gelu":
            zf = z.float()
            return (0.5 * zf * (1.0 + torch.erf(zf * (1.0 / math.sqrt(2.0))))).to(out_dtype)
        if kind != "tanh":
            raise ValueError(kind)
        return torch.tanh(z.float()).to(out_dtype)

    def unfolded_attention_ok(self, dk, dv, cdt):
        """Whether a prompt's attention with per-head keys of size dk and values of size dv is worth
        materialising them (here: always, so that the CPU path runs both forms)."""
        return True

    def head_matmul_nt(self, a, w, heads, a_stride, out, out_stride):
        """Per head h: out[:, h * out_stride : + N] = a[:, h * a_stride : + K] . w[h]^T  (w: [heads, N, K]);
        the operands are rounded to w's type, the fp32 accumulator to out's."""
        _, N, K = w.shape
        T = a.shape[0]
        av = torch.stack([a[:, h * a_stride:h * a_stride + K] for h in range(heads)], 1).to(w.dtype).float()
        y = torch.einsum("thk,hnk->thn", av, w.float())
        for h in range(heads):
            out[:, h * out_stride:h * out_stride + N] = y[:, h].to(out.dtype)
        return out

    @staticmethod
    def rope_freqs(dims, base, device, scaling=None):
        """f_i = base^(-2i / dims), i < dims / 2, rounded once to fp32.  ``scaling`` = (factor, low, high,
        original): a frequency whose wavelength 2 pi / f is longer than original / low is divided by
        factor, one shorter than original / high stays, and between them the two are blended linearly in
        s = (original / wavelength - low) / (high - low)."""
        i = torch.arange(dims // 2, dtype=torch.float64)
        f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * i / dims)
        if scaling is not None and scaling[0] == "turns":
            # ("turns", factor, original, fast, slow): by the entry number at which a pair makes ``fast`` /
            # ``slow`` turns over ``original`` positions, e(t) = dims ln(original / (2 pi t)) / (2 ln base):
            # entries up to lo = floor(e(fast)) keep their frequency, from hi = ceil(e(slow)) on they are
            # divided by factor, a linear ramp between
            factor, orig, fast, slow = (float(v) for v in scaling[1:])
            e = lambda t: dims * math.log(orig / (2 * math.pi * t)) / (2 * math.log(float(base)))
            lo, hi = max(math.floor(e(fast)), 0), min(math.ceil(e(slow)), dims - 1)
            ramp = torch.clamp((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
            f = f / factor * ramp + f * (1 - ramp)
        elif scaling is not None:
            factor, low, high, orig = (float(v) for v in scaling)
            wl = 2 * math.pi / f
            s_ = (orig / wl - low) / (high - low) if high != low else torch.ones_like(f)
            mid = (1 - s_) * f / factor + s_ * f
            f = torch.where(wl < orig / high, f, torch.where(wl > orig / low, f / factor, mid))
        return f.float().to(device)

    @staticmethod
    def rope_amp(scaling) -> float:
        """The factor on every cosine and sine: 0.1 ln(factor) + 1 for the ("turns", ...) rescaling, else 1."""
        if scaling is not None and scaling[0] == "turns":
            return 0.1 * math.log(float(scaling[1])) + 1.0
        return 1.0

    def head_norm_rope(self, x, heads, n, x_col, x_hs, out, out_col, out_hs, meta, w=None, eps=0.0, rot=None,
                       row_map=None, raw=None, unit_after=False, half=False):
        """Per row t and head h the n entries x[t, x_col + h * x_hs : + n]: RMS-normed over n times w
        (when w is given), then the first rot = (dims, base[, scaling])[0] entries rotated in pairs
        (2i, 2i + 1) -- with ``half`` in pairs (i, i + dims / 2) -- by the angle pos_t * f_i (``rope_freqs``,
        cosine and sine times ``rope_amp``), then, with ``unit_after``, divided by
        their root mean square over n (eps inside the root, no weight); written to
        out[row, out_col + h * out_hs : + n], row = t or row_map[t].  ``raw``: a matrix like out that
        receives the entries as they came."""
        T = x.shape[0]
        v = torch.stack([x[:, x_col + h * x_hs:x_col + h * x_hs + n] for h in range(heads)], 1).float()    # [T, heads, n]
        keep = v.clone()
        if w is not None:
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps) * w.float()
        if rot is not None and rot[0] > 0:
            dims, base = rot[0], rot[1]
            sc = rot[2] if len(rot) > 2 else None
            freqs = self.rope_freqs(dims, base, x.device, sc)
            ang = meta["tok_pos"].float()[:, None] * freqs[None, :]                                     # fp32 angles
            amp = self.rope_amp(sc)
            c, s_ = amp * torch.cos(ang)[:, None, :], amp * torch.sin(ang)[:, None, :]
            ia, ib = (slice(0, dims // 2), slice(dims // 2, dims)) if half else (slice(0, dims, 2), slice(1, dims, 2))
            a, b = v[:, :, ia], v[:, :, ib]
            r = v.clone()
            r[:, :, ia] = a * c - b * s_
            r[:, :, ib] = b * c + a * s_
            v = r
        if unit_after:
            v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
        rows = row_map.long() if row_map is not None else torch.arange(T, device=x.device)
        for h in range(heads):
            out[rows, out_col + h * out_hs:out_col + h * out_hs + n] = v[:, h].to(out.dtype)
            if raw is not None:
                raw[rows, out_col + h * out_hs:out_col + h * out_hs + n] = keep[:, h].to(raw.dtype)
        return out

    def qkv_conv_rope_store(self, z, w, state, meta, H, G, d, dv, q_out, kc, vc, eps=0.0, rot=None, v_heads=None, q_norm=None,
                            k_norm=None):
        """The projected rows z = [q (H d) | k (G d) | v (G dv) | ...] of a step on their way into attention:
        a short causal convolution per channel (``w`` [C, taps], no bias; the last taps - 1 rows of a request
        carried in ``state[slot]``, None for one tap), then for q and k heads the pair rotation ``rot`` and
        the division by the head's root mean square (eps inside the root), v as convolved.  q goes to
        ``q_out`` [T, H d] fp32, k and v to the rows ``kv_slot`` of their pools.  G = 0 (kc, vc None): a layer
        that reads another layer's keys and values has only queries.  ``v_heads``: the row holds that many value
        heads (instead of G) behind its G key heads.  ``q_norm`` / ``k_norm`` ([d]): the q / k heads are instead
        RMS-normed before the rotation and multiplied by that weight."""
        Gv = G if v_heads is None else int(v_heads)
        C = H * d + G * d + Gv * dv
        u = z[:, :C]
        if w is not None:
            if w.shape[1] > 1:
                u = self.causal_conv(u, w, None, state, meta)
            else:
                u = u.float() * w.float()[:, 0]
        self.head_norm_rope(u, H, d, 0, d, q_out, 0, d, meta, w=q_norm, eps=eps, rot=rot, unit_after=q_norm is None)
        if G:
            self.head_norm_rope(u, G, d, H * d, d, kc.view(-1, kc.shape[-1]), 0, d, meta, w=k_norm, eps=eps, rot=rot,
                                unit_after=k_norm is None, row_map=meta["kv_slot"])
            self.head_norm_rope(u, Gv, dv, (H + G) * d, dv, vc.view(-1, vc.shape[-1]), 0, dv, meta, row_map=meta["kv_slot"])
        return q_out

    def softcap_(self, z, cap):
        z.copy_(cap * torch.tanh(z / cap))
        return z

    def gather_rows(self, x, idx, out=None):
        return x.index_select(0, idx.long())

    # ------------------------------------------------------------- attention
    def kv_store(self, k, kn, eps, v, kcache, vcache, kv_slot):
        """k rows RMS-normed over their whole width (times kn), then k and v written to their places."""
        kf = k.float()
        kf = kf * torch.rsqrt(kf.pow(2).mean(-1, keepdim=True) + eps) * kn.float()
        kcache.view(-1, kcache.shape[-1]).index_copy_(0, kv_slot.long(), kf.to(kcache.dtype))
        vcache.view(-1, vcache.shape[-1]).index_copy_(0, kv_slot.long(), v.to(vcache.dtype))

    def attn_paged(self, q, kcache, vcache, meta, H, G, d, dv, scale, softcap, r1, r2, chunk, page_size, out_dtype,
                   window=0, keep_first=0, gate_bias=None, out_scale=1.0, out=None, sink=None, head_gate=None, v_heads=None):
        """Row i of a request sees the keys j <= i of its own chunk (``chunk`` > 0: floor(i / chunk) ==
        floor(j / chunk)) or window (``window`` > 0: j > i - window, and besides them the first
        ``keep_first`` keys of the sequence), read from the request's pages.  Head h of H reads key /
        value head h // (H / G): the first G * d (G * dv) columns of a pool row.  Weights: softmax over
        the visible keys of cap(scale q.k) - r1 log(1 + r2 (i - j)), or, with ``gate_bias`` [H],
        sigmoid(scale q.k + gate_bias[h]) for each key by itself.  ``sink`` (a number): the softmax has one
        more entry of that score and no value, p_j = exp(s_j) / (exp(sink) + sum exp(s)).  ``head_gate``
        [T, H] fp32: head h's output of row t times sigmoid(head_gate[t, h]).  The result times ``out_scale``.
        ``v_heads`` (a divisor of G): the pool holds only that many value heads, key head g reads value
        head g % v_heads (several score maps over the same values).  ``out`` may be fp32 over bf16 pools."""
        T = q.shape[0]
        res = torch.empty(T, H * dv, dtype=torch.float32, device=q.device)
        kf = kcache.reshape(-1, kcache.shape[-1])[:, :G * d].reshape(-1, G, d)
        Gv = int(v_heads or G)
        vf = vcache.reshape(-1, vcache.shape[-1])[:, :Gv * dv].reshape(-1, Gv, dv)
        if Gv != G:
            vf = vf.repeat(1, G // Gv, 1)
        qf = q.float().view(T, H, d)
        pos, seq, table = meta["tok_pos"].tolist(), meta["tok_seq"].tolist(), meta["page_table"]
        rep = H // G
        for t in range(T):
            i = pos[t]
            lo = (i // chunk) * chunk if chunk > 0 else 0
            if window > 0:
                lo = max(lo, i - window + 1)
            js = torch.arange(lo, i + 1, device=q.device)
            if keep_first > 0 and lo > 0:
                js = torch.cat([torch.arange(0, min(keep_first, lo), device=q.device), js])
            rows = table[seq[t]].long()[js // page_size] * page_size + js % page_size
            kk, vv = kf[rows].float(), vf[rows].float()            # [n, G, d]
            s = torch.einsum("hd,nhd->hn", qf[t], kk.repeat_interleave(rep, 1)) * scale
            if softcap > 0:
                s = softcap * torch.tanh(s / softcap)
            if r1 is not None:
                s = s - r1.float()[:, None] * torch.log1p(r2.float()[:, None] * (i - js).float()[None, :])
            if gate_bias is not None:
                p = torch.sigmoid(s + gate_bias.float()[:, None])
            elif sink is not None:
                p = torch.softmax(torch.cat([s, torch.full((H, 1), float(sink), device=q.device)], -1), -1)[:, :-1]
            else:
                p = torch.softmax(s, -1)
            o = torch.einsum("hn,nhv->hv", p, vv.repeat_interleave(rep, 1))
            if head_gate is not None:
                o = o * torch.sigmoid(head_gate[t].float())[:, None]
            res[t] = o.reshape(-1) * out_scale
        if out is not None:
            out.copy_(res.to(out.dtype))
            return out
        return res.to(out_dtype)

    # ------------------------------------------------------------ recurrences
    def causal_conv(self, x, w, b, state, meta, act="none", residual=False, out_dtype=torch.float32):
        """Per channel and request: out_t = b + sum_j w[:, taps-1-j] x_(t-j) (+ x_t with ``residual``;
        ``b`` may be None); inputs before this step's rows come from ``state[slot]`` (the last taps-1
        inputs), zeros before position 0.  The state is updated to the last taps-1 inputs after this step."""
        T, C = x.shape
        taps = w.shape[1]
        out = torch.empty(T, C, dtype=torch.float32, device=x.device)
        cu, pos0, slot = meta["cu_host"], meta["pos0_host"], meta["slot"].tolist()
        wf, xf = w.float(), x.float()
        for s in range(len(slot)):
            a, e = int(cu[s]), int(cu[s + 1])
            hist = state[slot[s]].clone() if pos0[s] > 0 else torch.zeros(taps - 1, C, device=x.device)
            full = torch.cat([hist, xf[a:e]], 0)                   # [taps-1 + n, C]
            n = e - a
            o = b.float().expand(n, C).clone() if b is not None else torch.zeros(n, C, device=x.device)
            for j in range(taps):
                o += wf[:, taps - 1 - j] * full[taps - 1 - j: taps - 1 - j + n]
            out[a:e] = o + xf[a:e] if residual else o
            if taps > 1:
                state[slot[s]] = full[-(taps - 1):]
        return (F.silu(out) if act == "silu" else out).to(out_dtype)

    def delta_rule_scan(self, r, k, v, a, wz, g, w0, norm_w, state, meta, heads, dim, decay_scale, key_eps, norm_eps,
                        out_scale, out):
        """Per head a state S [key channel, value channel], carried in ``state[slot]``:
        S_t = diag(w_t) S_(t-1) - (a_t * u_t)(u_t^T S_(t-1)) + k_t v_t^T,   o_t = S_t^T r_t,
        u = k / sqrt(sum(k^2) + key_eps), w = exp(-decay_scale sigmoid(wz + w0)), a = sigmoid(a);
        out = out_scale * o / sqrt(mean_head(o^2) + norm_eps) * norm_w * sigmoid(g)."""
        T = r.shape[0]
        H, d = heads, dim
        sh = lambda t: t.float().reshape(T, H, d)
        rr, kk, vv = sh(r), sh(k), sh(v)
        w = torch.exp(-decay_scale * torch.sigmoid(wz.float() + w0.float())).reshape(T, H, d)
        aa = torch.sigmoid(a.float()).reshape(T, H, d)
        u = kk * torch.rsqrt(kk.pow(2).sum(-1, keepdim=True) + key_eps)
        o = torch.empty(T, H, d, dtype=torch.float32, device=r.device)
        cu, pos0, slot = meta["cu_host"], meta["pos0_host"], meta["slot"].tolist()
        for s in range(len(slot)):
            S = state[slot[s]].clone() if pos0[s] > 0 else torch.zeros(H, d, d, device=r.device)
            for t in range(int(cu[s]), int(cu[s + 1])):
                uS = torch.einsum("hk,hkv->hv", u[t], S)
                S = w[t][:, :, None] * S - (aa[t] * u[t])[:, :, None] * uS[:, None, :] + kk[t][:, :, None] * vv[t][:, None, :]
                o[t] = torch.einsum("hkv,hk->hv", S, rr[t])
            state[slot[s]] = S
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + norm_eps)
        y = o.reshape(T, H * d) * norm_w.float() * torch.sigmoid(g.float()) * out_scale
        out.copy_(y.to(out.dtype))
        return out

    def diff_combine(self, a, lam_w, diff, H, dv, eps, out_dtype):
        """a: [T, 2 H dv], the outputs of two score maps, all heads of the first map, then all of the second.
        Per head o = a1 - lambda a2 with lambda = exp(sum(lam_w[0] lam_w[1])) - exp(sum(lam_w[2] lam_w[3])) + diff,
        then o / sqrt(mean(o^2) + eps) * (1 - diff)."""
        T = a.shape[0]
        lw = lam_w.float()
        lam = torch.exp((lw[0] * lw[1]).sum()) - torch.exp((lw[2] * lw[3]).sum()) + float(diff)
        a3 = a.float().reshape(T, 2, H, dv)
        o = a3[:, 0] - lam * a3[:, 1]
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * (1.0 - float(diff))
        return o.reshape(T, H * dv).to(out_dtype)

    def hgrn2_scan(self, q, f, v, fb, lower, norm_w, state, meta, heads, dim, vdim, eps, out_dtype):
        """Per head a state S [dim, vdim] carried in ``state[slot]``: with the forget gate
        g_t = lower + (1 - lower) sigmoid(f_t + fb) per state row,  S_t = diag(g_t) S_(t-1) + (1 - g_t) v_t^T,
        o_t = S_t^T silu(q_t); returns o / sqrt(mean_head(o^2) + eps) * norm_w (norm_w [vdim], shared by the heads)."""
        T, H = q.shape[0], heads
        qq = F.silu(q.float()).reshape(T, H, dim)
        lo = lower.float()
        ff = f.float() + fb.float() if fb is not None else f.float()      # (fb None: the bias is already in f)
        gg = (lo + (1 - lo) * torch.sigmoid(ff)).reshape(T, H, dim)
        vv = v.float().reshape(T, H, vdim)
        o = torch.empty(T, H, vdim, dtype=torch.float32, device=q.device)
        cu, pos0, slot = meta["cu_host"], meta["pos0_host"], meta["slot"].tolist()
        for s in range(len(slot)):
            S = state[slot[s]].clone() if pos0[s] > 0 else torch.zeros(H, dim, vdim, device=q.device)
            for t in range(int(cu[s]), int(cu[s + 1])):
                S = gg[t][:, :, None] * S + (1 - gg[t])[:, :, None] * vv[t][:, None, :]
                o[t] = torch.einsum("hkv,hk->hv", S, qq[t])
            state[slot[s]] = S
        o = o * torch.rsqrt(o.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
        return o.reshape(T, H * vdim).to(out_dtype)

    def rglru_scan(self, u, g, lam, y, state, meta, c, out_dtype):
        """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) sigmoid(g_i) u_t,  a_t = exp(-c sigmoid(g_r) softplus(lam));
        returns S_t * gelu_tanh(y_t)."""
        T, Wd = u.shape
        r, ig = torch.sigmoid(g[:, :Wd].float()), torch.sigmoid(g[:, Wd:].float())
        a = torch.exp(-c * r * F.softplus(lam.float()))
        inp = torch.sqrt(1 - a * a) * ig * u.float()
        out = torch.empty(T, Wd, dtype=torch.float32, device=u.device)
        cu, pos0, slot = meta["cu_host"], meta["pos0_host"], meta["slot"].tolist()
        for s in range(len(slot)):
            S = state[slot[s]].clone() if pos0[s] > 0 else torch.zeros(Wd, device=u.device)
            for t in range(int(cu[s]), int(cu[s + 1])):
                S = a[t] * S + inp[t]
                out[t] = S
            state[slot[s]] = S
        yf = y.float()
        gelu = 0.5 * yf * (1 + torch.tanh(math.sqrt(2 / math.pi) * (yf + 0.044715 * yf ** 3)))
        return (out * gelu).to(out_dtype)

    def ssd_scan(self, xbc, z, dt, dt_bias, A_log, Dskip, state, meta, nh, P, N, G):
        """Per head: S_t = exp(-exp(A) dt_t) S_(t-1) + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t with
        dt_t = softplus(dt_t + dt_bias); returns y * silu(z) as fp32 [T, nh * P]."""
        T = xbc.shape[0]
        inner = nh * P
        x = xbc[:, :inner].float().reshape(T, nh, P)
        B = xbc[:, inner:inner + G * N].float().reshape(T, G, N).repeat_interleave(nh // G, 1)
        C = xbc[:, inner + G * N:].float().reshape(T, G, N).repeat_interleave(nh // G, 1)
        dtv = F.softplus(dt.float() + dt_bias.float())                      # [T, nh]
        dec = torch.exp(-torch.exp(A_log.float()) * dtv)
        out = torch.empty(T, nh, P, dtype=torch.float32, device=xbc.device)
        cu, pos0, slot = meta["cu_host"], meta["pos0_host"], meta["slot"].tolist()
        for s in range(len(slot)):
            S = state[slot[s]].clone() if pos0[s] > 0 else torch.zeros(nh, N, P, device=xbc.device)
            for t in range(int(cu[s]), int(cu[s + 1])):
                S = dec[t][:, None, None] * S + dtv[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
                out[t] = torch.einsum("hnp,hn->hp", S, C[t]) + Dskip.float()[:, None] * x[t]
            state[slot[s]] = S
        zf = z.float()
        return out.reshape(T, inner) * (zf * torch.sigmoid(zf))

    # ------------------------------------------------------ mixture of experts
    def moe_route_corrected(self, logits, corr, top):
        """softmax over the experts; the ``top`` largest of (score + corr) are chosen (ties: the lower
        expert), each weighted by its bare score."""
        T, E = logits.shape
        s = torch.softmax(logits.float(), -1)
        choice = s + corr.float()
        ids = torch.sort(choice, dim=-1, descending=True, stable=True).indices[:, :top]
        w = s.gather(1, ids)
        flat = ids.reshape(-1)
        order = torch.sort(flat, stable=True).indices
        dest = torch.empty_like(order)
        dest[order] = torch.arange(order.numel(), device=order.device)
        offs = torch.zeros(E + 1, dtype=torch.int32, device=logits.device)
        offs[1:] = torch.cumsum(torch.bincount(flat, minlength=E), 0)
        return SeqRoute(ids.int(), w, offs, (order // top).int(), dest.int().reshape(T, top), top)

    def moe_route_topk(self, logits, top):
        """The ``top`` largest logits are chosen (ties: the lower expert), weighted by the softmax over
        the chosen logits only."""
        T, E = logits.shape
        vals, ids = torch.sort(logits.float(), dim=-1, descending=True, stable=True)
        ids, w = ids[:, :top], torch.softmax(vals[:, :top], -1)
        flat = ids.reshape(-1)
        order = torch.sort(flat, stable=True).indices
        dest = torch.empty_like(order)
        dest[order] = torch.arange(order.numel(), device=order.device)
        offs = torch.zeros(E + 1, dtype=torch.int32, device=logits.device)
        offs[1:] = torch.cumsum(torch.bincount(flat, minlength=E), 0)
        return SeqRoute(ids.int(), w, offs, (order // top).int(), dest.int().reshape(T, top), top)

    def moe_route_grouped(self, logits, top, groups, keep, scale):
        """Scores sigmoid(logit).  The experts form ``groups`` equal groups of neighbours, a group is worth the
        sum of its two largest scores, and only experts of the ``keep`` best groups compete (``groups`` 0 or
        1: all do).  The ``top`` largest scores are chosen (ties: the lower expert), weighted by
        score / (sum of the chosen + 1e-20) * scale."""
        T, E = logits.shape
        sc = torch.sigmoid(logits.float())
        cand = sc
        if groups and groups > 1:
            per = E // groups
            worth = torch.sort(sc.reshape(T, groups, per), dim=-1, descending=True).values[:, :, :2].sum(-1)
            kept = torch.sort(worth, dim=-1, descending=True, stable=True).indices[:, :keep]
            ok = torch.zeros(T, groups, dtype=torch.bool, device=logits.device)
            ok.scatter_(1, kept, True)
            cand = torch.where(ok.repeat_interleave(per, 1), sc, torch.full_like(sc, -1.0))
        ids = torch.sort(cand, dim=-1, descending=True, stable=True).indices[:, :top]
        w = sc.gather(1, ids)
        w = w / (w.sum(-1, keepdim=True) + 1e-20) * float(scale)
        flat = ids.reshape(-1)
        order = torch.sort(flat, stable=True).indices
        dest = torch.empty_like(order)
        dest[order] = torch.arange(order.numel(), device=order.device)
        offs = torch.zeros(E + 1, dtype=torch.int32, device=logits.device)
        offs[1:] = torch.cumsum(torch.bincount(flat, minlength=E), 0)
        return SeqRoute(ids.int(), w, offs, (order // top).int(), dest.int().reshape(T, top), top)

    def grouped_matmul_nt(self, a, w, offs):
        E, N, K = w.shape
        out = torch.zeros(a.shape[0], N, dtype=torch.float32, device=a.device)
        o = offs.tolist()
        for e in range(E):
            if o[e + 1] > o[e]:
                out[o[e]:o[e + 1]] = self.matmul_nt(a[o[e]:o[e + 1]], w[e])
        return out

    def moe_weighted_sum(self, y, route):
        T, top = route.dest.shape
        return (y[route.dest.long().reshape(-1)].reshape(T, top, -1) * route.w[:, :, None]).sum(1)

    def moe_combine_(self, x, y, route, mult, shared=None, shared_gate=None):
        """x += mult * (sum_k w[t, k] y[dest[t, k]] + sigmoid(shared_gate[t]) * shared[t]): the experts'
        weighted sum, the gated shared expert (both optional parts fp32; ``shared_gate`` [T, 1]) and the
        residual update in one pass."""
        s = self.moe_weighted_sum(y, route)
        if shared is not None:
            g = torch.sigmoid(shared_gate.float()) if shared_gate is not None else 1.0
            s = s + g * shared.float()
        x.add_(s, alpha=float(mult))
        return x

    def argmax_f32(self, z):
        return z.argmax(-1).int()
