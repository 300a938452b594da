"""HIP ops of the stateful (hybrid) models: the kernels of ``csrc/kernels/seq`` (``libfls_seq.so``)
behind the signatures of :class:`~.torch_seq.TorchSeqOps`.

Every kernel runs on the caller's current HIP stream; outputs come from PyTorch's caching allocator.
There is no fallback: a missing library raises.  Norms, scores, softmax, gates, recurrences and the
residual stream are fp32 in both modes; ``out_dtype`` (bf16 or fp32) is the element type of what the
next matrix product reads, and a product returns its fp32 accumulator.
"""
from __future__ import annotations

import torch

from .. import _native
from .torch_seq import SeqRoute

_CODE = {torch.float32: 0, torch.bfloat16: 1}


def _stream():
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def _chk(rc: int, what: str):
    if rc != 0:
        raise RuntimeError(f"{what} failed with code {rc}")


def _code(t: torch.Tensor, name: str) -> int:
    if t.dtype not in _CODE or not t.is_cuda:
        raise TypeError(f"{name}: expected an fp32 or bf16 CUDA tensor, got {t.dtype} on {t.device}")
    return _CODE[t.dtype]


def _rows(t: torch.Tensor, name: str, dtype=None):
    """A 2-D tensor with unit column stride (a column slice of a wider buffer is fine)."""
    if t.dim() != 2 or (t.shape[1] > 1 and t.stride(1) != 1) or not t.is_cuda:
        raise ValueError(f"{name}: expected a CUDA matrix with contiguous rows, got {tuple(t.shape)} / {t.stride()}")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    return t


def _vec(t: torch.Tensor, name: str, n: int, dtype=torch.float32):
    if t.dtype != dtype or not t.is_cuda or not t.is_contiguous() or t.numel() != n:
        raise TypeError(f"{name}: expected a contiguous {dtype} CUDA tensor of {n} elements, got {t.dtype} {tuple(t.shape)}")
    return t


class HipSeqOps:
    name = "hip-seq"
    fused_norm = False

    def __init__(self):
        self.k = _native.seq_kernels()
        self._freqs = {}

    # ----------------------------------------------------------------- rows
    def embed_rows(self, ids, table, out=None, scale=1.0, pos_table=None, tok_pos=None, copies=1):
        T, (V, D) = ids.numel(), table.shape
        if out is None:
            out = torch.empty(T, D * copies, dtype=torch.float32, device=table.device)
        if out.dtype != torch.float32 or not out.is_contiguous() or tuple(out.shape) != (T, D * copies):
            raise TypeError("embed_rows: out must be a contiguous fp32 [T, copies * D] tensor")
        _vec(ids, "ids", T, torch.int32)
        if pos_table is not None or copies != 1:
            if pos_table is not None:
                if pos_table.dtype != table.dtype or pos_table.shape[1] != D or not pos_table.is_contiguous() or not table.is_contiguous():
                    raise TypeError("embed_rows: pos_table must be laid out like table")
                _vec(tok_pos, "tok_pos", T, torch.int32)
            _chk(self.k.fls_seq_embed_pos(ids.data_ptr(), table.data_ptr(), _code(table, "table"),
                                          pos_table.data_ptr() if pos_table is not None else None,
                                          tok_pos.data_ptr() if pos_table is not None else None, out.data_ptr(), T, D, V,
                                          pos_table.shape[0] if pos_table is not None else 0, float(scale), int(copies), _stream()),
                 "fls_seq_embed_pos")
            return out
        _chk(self.k.fls_seq_embed(ids.data_ptr(), table.data_ptr(), _code(table, "table"), out.data_ptr(), T, D, V,
                                  float(scale), _stream()), "fls_seq_embed")
        return out

    def group_rmsnorm(self, x, w, groups, eps, out_dtype, row_idx=None, w_offset=0.0):
        _rows(x, "x", torch.float32)
        rows = x.shape[0] if row_idx is None else row_idx.numel()
        D = x.shape[1]
        _vec(w, "w", D)
        if row_idx is not None:
            _vec(row_idx, "row_idx", rows, torch.int32)
        y = torch.empty(rows, D, dtype=out_dtype, device=x.device)
        _chk(self.k.fls_seq_group_rmsnorm(x.data_ptr(), x.stride(0), row_idx.data_ptr() if row_idx is not None else None,
                                          w.data_ptr(), y.data_ptr(), _CODE[out_dtype], D, rows, D, groups, float(eps), 0,
                                          float(w_offset), _stream()), "fls_seq_group_rmsnorm")
        return y

    def add_group_rmsnorm_(self, x, y, w, groups, eps, w_offset=0.0):
        _rows(x, "x", torch.float32)
        _rows(y, "y", torch.float32)
        if x.shape != y.shape:
            raise ValueError("add_group_rmsnorm_: shapes differ")
        _vec(w, "w", x.shape[1])
        _chk(self.k.fls_seq_group_rmsnorm(y.data_ptr(), y.stride(0), None, w.data_ptr(), x.data_ptr(), 0, x.stride(0),
                                          x.shape[0], x.shape[1], groups, float(eps), 1, float(w_offset), _stream()),
             "fls_seq_group_rmsnorm")
        return x

    def dyt_norm(self, x, wb, alpha, out_dtype, row_idx=None):
        _rows(x, "x", torch.float32)
        rows = x.shape[0] if row_idx is None else row_idx.numel()
        D = x.shape[1]
        _vec(wb, "wb", 2 * D)
        _vec(alpha, "alpha", 1)
        if row_idx is not None:
            _vec(row_idx, "row_idx", rows, torch.int32)
        y = torch.empty(rows, D, dtype=out_dtype, device=x.device)
        _chk(self.k.fls_seq_dyt_norm(x.data_ptr(), x.stride(0), row_idx.data_ptr() if row_idx is not None else None,
                                     wb.data_ptr(), alpha.data_ptr(), y.data_ptr(), _CODE[out_dtype], D, rows, D, _stream()),
             "fls_seq_dyt_norm")
        return y

    def add_scaled_(self, x, y, mult):
        _rows(x, "x", torch.float32)
        _rows(y, "y", torch.float32)
        if x.shape != y.shape:
            raise ValueError("add_scaled_: shapes differ")
        _chk(self.k.fls_seq_add_scaled(x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0), x.shape[0], x.shape[1],
                                       float(mult), _stream()), "fls_seq_add_scaled")
        return x

    def add_scaled_dyt_norm_(self, x, y, mult, wb, alpha, out_dtype):
        _rows(x, "x", torch.float32)
        _rows(y, "y", torch.float32)
        if x.shape != y.shape:
            raise ValueError("add_scaled_dyt_norm_: shapes differ")
        T, D = x.shape
        _vec(wb, "wb", 2 * D)
        _vec(alpha, "alpha", 1)
        h = torch.empty(T, D, dtype=out_dtype, device=x.device)
        _chk(self.k.fls_seq_add_scaled_dyt(x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0), float(mult), wb.data_ptr(),
                                           alpha.data_ptr(), h.data_ptr(), _CODE[out_dtype], D, T, D, _stream()),
             "fls_seq_add_scaled_dyt")
        return h

    def streams_norm(self, xs, coef, w, eps, out_dtype, streams, row_idx=None):
        _rows(xs, "xs", torch.float32)
        D = xs.shape[1] // streams
        if xs.shape[1] != streams * D:
            raise ValueError("streams_norm: the row is not streams * D wide")
        rows = xs.shape[0] if row_idx is None else row_idx.numel()
        _vec(w, "w", D)
        if coef is not None and (coef.dtype != torch.float32 or not coef.is_contiguous() or coef.numel() < streams):
            raise TypeError("streams_norm: coef must be fp32 with at least one entry per stream")
        if row_idx is not None:
            _vec(row_idx, "row_idx", rows, torch.int32)
        y = torch.empty(rows, D, dtype=out_dtype, device=xs.device)
        _chk(self.k.fls_seq_streams_norm(xs.data_ptr(), xs.stride(0), row_idx.data_ptr() if row_idx is not None else None,
                                         coef.data_ptr() if coef is not None else None, w.data_ptr(), y.data_ptr(),
                                         _CODE[out_dtype], D, rows, D, streams, float(eps), _stream()), "fls_seq_streams_norm")
        return y

    def _streams_update(self, xs, y, gate, hc, mult, streams, coef, w, eps, out_dtype):
        _rows(xs, "xs", torch.float32)
        _rows(y, "y", torch.float32)
        T, D = y.shape
        if tuple(xs.shape) != (T, streams * D):
            raise ValueError("streams_update_: xs must be [T, streams * D]")
        if gate is not None:
            _rows(gate, "gate", torch.float32)
            if tuple(gate.shape) != (T, D):
                raise ValueError("streams_update_: gate is [T, D]")
        if hc is not None:
            _vec(hc, "hc", 2 * streams + streams * streams)
        elif streams != 1:
            raise ValueError("streams_update_: several streams need their coefficients")
        h = None
        if w is not None:
            _vec(w, "w", D)
            if coef is not None and (coef.dtype != torch.float32 or not coef.is_contiguous() or coef.numel() < streams):
                raise TypeError("streams_update_norm_: coef must be fp32 with at least one entry per stream")
            h = torch.empty(T, D, dtype=out_dtype, device=xs.device)
        _chk(self.k.fls_seq_streams_update(xs.data_ptr(), xs.stride(0), y.data_ptr(), y.stride(0),
                                           gate.data_ptr() if gate is not None else None, gate.stride(0) if gate is not None else 0,
                                           hc.data_ptr() if hc is not None else None, float(mult), T, D, streams,
                                           coef.data_ptr() if (w is not None and coef is not None) else None,
                                           w.data_ptr() if w is not None else None, h.data_ptr() if h is not None else None,
                                           _CODE[out_dtype] if h is not None else 0, D, float(eps), _stream()),
             "fls_seq_streams_update")
        return h

    def streams_update_(self, xs, y, gate, hc, mult, streams):
        self._streams_update(xs, y, gate, hc, mult, streams, None, None, 0.0, torch.float32)
        return xs

    def streams_update_norm_(self, xs, y, gate, hc, mult, streams, coef, w, eps, out_dtype):
        return self._streams_update(xs, y, gate, hc, mult, streams, coef, w, eps, out_dtype)

    def scale_(self, z, alpha):
        _rows(z, "z", torch.float32)
        _chk(self.k.fls_seq_scale(z.data_ptr(), z.stride(0), z.shape[0], z.shape[1], float(alpha), _stream()), "fls_seq_scale")
        return z

    def sigmoid_gate(self, o, g, out_dtype):
        _rows(o, "o")
        _rows(g, "g", torch.float32)
        if o.shape != g.shape:
            raise ValueError("sigmoid_gate: shapes differ")
        y = torch.empty(o.shape, dtype=out_dtype, device=o.device)
        _chk(self.k.fls_seq_sigmoid_gate(o.data_ptr(), _code(o, "o"), o.stride(0), g.data_ptr(), g.stride(0), y.data_ptr(),
                                         _CODE[out_dtype], y.stride(0), o.shape[0], o.shape[1], _stream()), "fls_seq_sigmoid_gate")
        return y

    def diff_combine(self, a, lam_w, diff, H, dv, eps, out_dtype):
        _rows(a, "a", torch.float32)
        if a.shape[1] != 2 * H * dv or lam_w.dim() != 2 or lam_w.shape[0] != 4:
            raise ValueError("diff_combine: a is [T, 2 H dv], lam_w [4, d]")
        _vec(lam_w, "lam_w", lam_w.numel())
        out = torch.empty(a.shape[0], H * dv, dtype=out_dtype, device=a.device)
        _chk(self.k.fls_seq_diff_combine(a.data_ptr(), a.stride(0), lam_w.data_ptr(), lam_w.shape[1], float(diff), H, dv, float(eps),
                                         out.data_ptr(), _CODE[out_dtype], out.stride(0), a.shape[0], _stream()), "fls_seq_diff_combine")
        return out

    def hgrn2_scan(self, q, f, v, fb, lower, norm_w, state, meta, heads, dim, vdim, eps, out_dtype):
        T = q.shape[0]
        for nme, t, n in (("q", q, heads * dim), ("f", f, heads * dim), ("v", v, heads * vdim)):
            _rows(t, nme, torch.float32)
            if tuple(t.shape) != (T, n):
                raise ValueError(f"hgrn2_scan: {nme} is {tuple(t.shape)}, not {(T, n)}")
        _vec(lower, "lower", heads * dim)
        _vec(norm_w, "norm_w", vdim)
        if fb is not None:
            _vec(fb, "fb", heads * dim)
        if tuple(state.shape[1:]) != (heads, dim, vdim) or not state.is_contiguous() or state.dtype != torch.float32:
            raise ValueError("hgrn2_scan: state must be fp32 [slots, heads, dim, vdim]")
        raw = torch.empty(T, heads * vdim, dtype=torch.float32, device=q.device)
        _chk(self.k.fls_seq_hgrn2_scan(q.data_ptr(), q.stride(0), f.data_ptr(), f.stride(0), v.data_ptr(), v.stride(0),
                                       fb.data_ptr() if fb is not None else None, lower.data_ptr(), state.data_ptr(),
                                       raw.data_ptr(), raw.stride(0), meta["cu"].data_ptr(), meta["pos0"].data_ptr(),
                                       meta["slot"].data_ptr(), meta["n_seqs"], heads, dim, vdim, _stream()), "fls_seq_hgrn2_scan")
        out = torch.empty(T, heads * vdim, dtype=out_dtype, device=q.device)
        # every head's output over its own root mean square, times the weight the heads share
        return self.head_norm_rope(raw, heads, vdim, 0, vdim, out, 0, vdim, meta, w=norm_w, eps=eps)

    def moe_route_grouped(self, logits, top, groups, keep, scale):
        _rows(logits, "logits", torch.float32)
        T, E = logits.shape
        dev = logits.device
        ids = torch.empty(T, top, dtype=torch.int32, device=dev)
        w = torch.empty(T, top, dtype=torch.float32, device=dev)
        ints = torch.zeros(3 * E + 1, dtype=torch.int32, device=dev)          # hist | cursor | offs
        hist, cursor, offs = ints[:E], ints[E:2 * E], ints[2 * E:]
        dest = torch.empty(T, top, dtype=torch.int32, device=dev)
        rows = torch.empty(T * top, dtype=torch.int32, device=dev)
        s = _stream()
        _chk(self.k.fls_seq_moe_route_grouped(logits.data_ptr(), logits.stride(0), T, E, top, int(groups or 0), int(keep or 0),
                                              float(scale), ids.data_ptr(), w.data_ptr(), hist.data_ptr(), s), "fls_seq_moe_route_grouped")
        _chk(self.k.fls_seq_moe_scan(hist.data_ptr(), E, offs.data_ptr(), cursor.data_ptr(), s), "fls_seq_moe_scan")
        _chk(self.k.fls_seq_moe_place(ids.data_ptr(), T * top, top, cursor.data_ptr(), dest.data_ptr(), rows.data_ptr(), s),
             "fls_seq_moe_place")
        return SeqRoute(ids, w, offs, rows, dest, top)

    def qkv_conv_rope_store(self, z, w, state, meta, H, G, d, dv, q_out, kc, vc, eps=0.0, rot=None, v_heads=None, q_norm=None,
                            k_norm=None):
        _rows(z, "z", torch.float32)
        _rows(q_out, "q_out", torch.float32)
        T = z.shape[0]
        Gv = G if v_heads is None else int(v_heads)
        C = H * d + G * d + Gv * dv
        for nme, t in (("q_norm", q_norm), ("k_norm", k_norm)):
            if t is not None:
                _vec(t, nme, d)
        if (q_norm is None) != (k_norm is None) and G:
            raise ValueError("qkv_conv_rope_store: q_norm and k_norm come together")
        if z.shape[1] < C or tuple(q_out.shape) != (T, H * d):
            raise ValueError("qkv_conv_rope_store: rows do not fit the head sizes")
        taps = 1
        if w is not None:
            taps = w.shape[1]
            _vec(w, "w", C * taps)
            if taps > 1 and (state is None or state.dtype != torch.float32 or not state.is_contiguous()
                             or tuple(state.shape[1:]) != (taps - 1, C)):
                raise ValueError("qkv_conv_rope_store: state must be fp32 [slots, taps - 1, C]")
        tc = 0
        if G:
            if kc.dtype != vc.dtype or kc.shape[-1] < G * d or vc.shape[-1] < Gv * dv or not kc.is_contiguous() \
                    or not vc.is_contiguous():
                raise ValueError("qkv_conv_rope_store: pools do not fit the head sizes")
            tc = _code(kc, "kc")
            _vec(meta["kv_slot"], "kv_slot", T, torch.int32)
        dims, freqs = 0, None
        if rot is not None and rot[0] > 0:
            dims = int(rot[0])
            freqs = self.rope_freqs(dims, rot[1], z.device, rot[2] if len(rot) > 2 else None)
        _chk(self.k.fls_seq_qkv_conv_rope(z.data_ptr(), z.stride(0), w.data_ptr() if w is not None else None,
                                          state.data_ptr() if state is not None and taps > 1 else None, taps,
                                          meta["tok_seq"].data_ptr(), meta["tok_pos"].data_ptr(), meta["cu"].data_ptr(),
                                          meta["pos0"].data_ptr(), meta["slot"].data_ptr(),
                                          meta["kv_slot"].data_ptr() if G else None, T, meta["n_seqs"], H, G, d, dv, float(eps),
                                          freqs.data_ptr() if freqs is not None else None, dims, q_out.data_ptr(),
                                          q_out.stride(0), kc.data_ptr() if G else None, kc.shape[-1] if G else 0,
                                          vc.data_ptr() if G else None, vc.shape[-1] if G else 0, tc,
                                          1 if meta.get("max_rows") == 1 else 0, Gv,
                                          q_norm.data_ptr() if q_norm is not None else None,
                                          k_norm.data_ptr() if k_norm is not None else None, _stream()), "fls_seq_qkv_conv_rope")
        return q_out

    def _gemm(self, a, w, c, bias, M, N, K, lda, ldw, ldc, groups=1, offs=None, a_gs=0, a_mod=1, w_gs=0, c_gs=0,
              act=None):
        _chk(self.k.fls_seq_gemm(a.data_ptr(), _code(a, "a"), w.data_ptr(), _code(w, "w"), c.data_ptr(), _code(c, "c"),
                                 bias.data_ptr() if bias is not None else None,
                                 act.data_ptr() if act is not None else None, M, N, K, lda, ldw, ldc, groups,
                                 offs.data_ptr() if offs is not None else None, a_gs, a_mod, w_gs, c_gs, _stream()),
             "fls_seq_gemm")

    def matmul_nt(self, a, w, bias=None, xielu=None, out_dtype=torch.float32):
        """a . w^T (+ bias); ``xielu`` ({p, q}): that activation in the epilogue; ``out_dtype``: the
        accumulator as it is (fp32) or rounded for the next product (bf16)."""
        _rows(a, "a")
        _rows(w, "w")
        M, K = a.shape
        N, K2 = w.shape
        if K != K2:
            raise ValueError(f"matmul_nt: K mismatch {tuple(a.shape)} x {tuple(w.shape)}")
        if a.dtype == torch.bfloat16 and w.dtype == torch.float32:
            raise TypeError("matmul_nt: bf16 rows against fp32 weights")
        if bias is not None:
            _vec(bias, "bias", N)
        if xielu is not None:
            _vec(xielu, "xielu", 2)
        c = torch.empty(M, N, dtype=out_dtype, device=a.device)
        self._gemm(a, w, c, bias, M, N, K, a.stride(0), w.stride(0), N, act=xielu)
        return c

    def block_linear(self, u, w, b, blocks, cdt):
        _rows(u, "u", torch.float32)
        T, Wd = u.shape
        G, bw, bw2 = w.shape
        if bw != bw2 or blocks * bw != Wd or G % blocks or not w.is_contiguous():
            raise ValueError(f"block_linear: {tuple(u.shape)} against {tuple(w.shape)} in {blocks} blocks")
        _vec(b, "b", G * bw)
        c = torch.empty(T, G * bw, dtype=torch.float32, device=u.device)
        self._gemm(u, w, c, b, T, bw, bw, u.stride(0), bw, G * bw, groups=G, a_gs=bw, a_mod=blocks, w_gs=bw * bw, c_gs=bw)
        return c

    def grouped_matmul_nt(self, a, w, offs):
        _rows(a, "a")
        E, N, K = w.shape
        if a.shape[1] != K or not w.is_contiguous():
            raise ValueError(f"grouped_matmul_nt: {tuple(a.shape)} against {tuple(w.shape)}")
        _vec(offs, "offs", E + 1, torch.int32)
        M = a.shape[0]
        c = torch.empty(M, N, dtype=torch.float32, device=a.device)
        self._gemm(a, w, c, None, M, N, K, a.stride(0), K, N, groups=E, offs=offs, w_gs=N * K)
        return c

    def xielu(self, z, act, out_dtype):
        _rows(z, "z", torch.float32)
        _vec(act, "act", 2)
        y = torch.empty(z.shape, dtype=out_dtype, device=z.device)
        _chk(self.k.fls_seq_xielu(z.data_ptr(), z.stride(0), act.data_ptr(), y.data_ptr(), _CODE[out_dtype], z.shape[1],
                                  z.shape[0], z.shape[1], _stream()), "fls_seq_xielu")
        return y

    _ACT = {"silu": 0, "gelu_tanh": 1}
    HEAD_TILE_SHAPES = ((576, 512), (320, 256), (192, 128))    # (key row, value columns) of fls_seq_attn_heads

    def gate_mul(self, gu, out_dtype, act="silu"):
        _rows(gu, "gu", torch.float32)
        cols = gu.shape[1] // 2
        y = torch.empty(gu.shape[0], cols, dtype=out_dtype, device=gu.device)
        _chk(self.k.fls_seq_gate_mul(gu.data_ptr(), gu.stride(0), y.data_ptr(), _CODE[out_dtype], cols, gu.shape[0], cols,
                                     self._ACT[act], _stream()), "fls_seq_gate_mul")
        return y

    def silu_mul(self, gu, out_dtype):
        return self.gate_mul(gu, out_dtype, "silu")

    def unary(self, z, kind, out_dtype):
        _rows(z, "z", torch.float32)
        if kind not in ("tanh", "gelu"):
            raise ValueError(kind)
        y = torch.empty(z.shape, dtype=out_dtype, device=z.device)
        _chk(self.k.fls_seq_unary(z.data_ptr(), z.stride(0), y.data_ptr(), _CODE[out_dtype], z.shape[1], z.shape[0],
                                  z.shape[1], 1 if kind == "gelu" else 0, _stream()), "fls_seq_unary")
        return y

    def unfolded_attention_ok(self, dk, dv, cdt):
        """Per-head keys of size dk and values of size dv that the matrix-core prompt attention serves."""
        return cdt == torch.bfloat16 and dk in (64, 128) and dv in (64, 128)

    def head_matmul_nt(self, a, w, heads, a_stride, out, out_stride):
        """Per head h: out[:, h * out_stride : + N] = a[:, h * a_stride : + K] . w[h]^T  (w: [heads, N, K])."""
        _rows(a, "a")
        _rows(out, "out")
        hh, N, K = w.shape
        if hh != heads or not w.is_contiguous() or (heads - 1) * a_stride + K > a.shape[1] \
                or (heads - 1) * out_stride + N > out.shape[1] or out.shape[0] != a.shape[0]:
            raise ValueError(f"head_matmul_nt: {tuple(a.shape)} x {tuple(w.shape)} -> {tuple(out.shape)}")
        self._gemm(a, w, out, None, a.shape[0], N, K, a.stride(0), K, out.stride(0), groups=heads, a_gs=a_stride,
                   a_mod=heads, w_gs=N * K, c_gs=out_stride)
        return out

    def rope_freqs(self, dims, base, device, scaling=None):
        key = (int(dims), float(base), str(device), None if scaling is None else tuple(scaling))
        if key not in self._freqs:
            from .torch_seq import TorchSeqOps
            self._freqs[key] = TorchSeqOps.rope_freqs(int(dims), float(base), device, scaling)
        return self._freqs[key]

    def head_norm_rope(self, x, heads, n, x_col, x_hs, out, out_col, out_hs, meta, w=None, eps=0.0, rot=None,
                       row_map=None, raw=None, unit_after=False, half=False):
        _rows(x, "x")
        _rows(out, "out")
        T = x.shape[0]
        if x_col + (heads - 1) * x_hs + n > x.shape[1] or out_col + (heads - 1) * out_hs + n > out.shape[1]:
            raise ValueError("head_norm_rope: a head lies outside its row")
        if row_map is not None:
            _vec(row_map, "row_map", T, torch.int32)
        elif out.shape[0] != T:
            raise ValueError("head_norm_rope: out has other rows than x")
        if raw is not None and (raw.dtype != out.dtype or raw.shape != out.shape):
            _rows(raw, "raw")
            raise ValueError("head_norm_rope: raw must be laid out like out")
        if w is not None:
            _vec(w, "w", n)
        dims, freqs, amp = 0, None, 1.0
        if rot is not None and rot[0] > 0:
            from .torch_seq import TorchSeqOps
            dims = int(rot[0])
            sc = rot[2] if len(rot) > 2 else None
            freqs = self.rope_freqs(dims, rot[1], x.device, sc)
            amp = TorchSeqOps.rope_amp(sc)
        _chk(self.k.fls_seq_head_norm_rope(x.data_ptr(), _code(x, "x"), x.stride(0), x_col, x_hs, heads, n,
                                           w.data_ptr() if w is not None else None, float(eps),
                                           freqs.data_ptr() if freqs is not None else None, dims, meta["tok_pos"].data_ptr(),
                                           row_map.data_ptr() if row_map is not None else None, out.data_ptr(),
                                           _code(out, "out"), out.stride(0), out_col, out_hs,
                                           raw.data_ptr() if raw is not None else None,
                                           raw.stride(0) if raw is not None else 0, T, 1 if unit_after else 0,
                                           1 if half else 0, float(amp), _stream()),
             "fls_seq_head_norm_rope")
        return out

    def softcap_(self, z, cap):
        _rows(z, "z", torch.float32)
        _chk(self.k.fls_seq_softcap(z.data_ptr(), z.stride(0), z.shape[0], z.shape[1], float(cap), _stream()),
             "fls_seq_softcap")
        return z

    def argmax_f32(self, z):
        _rows(z, "z", torch.float32)
        out = torch.empty(z.shape[0], dtype=torch.int32, device=z.device)
        _chk(self.k.fls_seq_argmax(z.data_ptr(), z.stride(0), z.shape[0], z.shape[1], out.data_ptr(), _stream()),
             "fls_seq_argmax")
        return out

    def gather_rows(self, x, idx, out=None):
        _rows(x, "x")
        n = idx.numel()
        _vec(idx, "idx", n, torch.int32)
        y = torch.empty(n, x.shape[1], dtype=x.dtype, device=x.device)
        _chk(self.k.fls_seq_gather_rows(x.data_ptr(), _code(x, "x"), x.stride(0), idx.data_ptr(), y.data_ptr(), x.shape[1],
                                        n, x.shape[1], _stream()), "fls_seq_gather_rows")
        return y

    # ------------------------------------------------------------- attention
    def kv_store(self, k, kn, eps, v, kcache, vcache, kv_slot):
        _rows(k, "k", torch.float32)
        _rows(v, "v", torch.float32)
        rows, kcols, vcols = k.shape[0], k.shape[1], v.shape[1]
        if kcache.shape[-1] != kcols or vcache.shape[-1] != vcols or kcache.dtype != vcache.dtype \
                or not kcache.is_contiguous() or not vcache.is_contiguous():
            raise ValueError("kv_store: pools do not fit the rows")
        _vec(kn, "kn", kcols)
        _vec(kv_slot, "kv_slot", rows, torch.int32)
        _chk(self.k.fls_seq_kv_store(k.data_ptr(), k.stride(0), kn.data_ptr(), float(eps), v.data_ptr(), v.stride(0),
                                     kcache.data_ptr(), vcache.data_ptr(), _code(kcache, "kcache"), kv_slot.data_ptr(), rows,
                                     kcols, vcols, _stream()), "fls_seq_kv_store")

    def attn_paged(self, q, kcache, vcache, meta, H, G, d, dv, scale, softcap, r1, r2, chunk, page_size, out_dtype,
                   window=0, keep_first=0, gate_bias=None, out_scale=1.0, out=None, sink=None, head_gate=None, v_heads=None):
        _rows(q, "q")
        T = q.shape[0]
        if kcache.dtype != out_dtype or vcache.dtype != out_dtype or q.shape[1] != H * d \
                or (q.dtype != out_dtype and q.dtype != torch.float32):
            raise TypeError("attn_paged: the pools share one element type (out_dtype); q is [T, H d] of it or fp32")
        ldk, ldv = kcache.shape[-1], vcache.shape[-1]
        Gv = int(v_heads or G)
        if G % Gv:
            raise ValueError("attn_paged: v_heads must divide the key heads")
        if ldk < G * d or ldv < Gv * dv or kcache.shape[1] != page_size or not kcache.is_contiguous() \
                or not vcache.is_contiguous():
            raise ValueError("attn_paged: pools do not fit the head sizes")
        table = meta["page_table"]
        for nme, t in (("r1", r1), ("r2", r2), ("gate_bias", gate_bias)):
            if t is not None:
                _vec(t, nme, H)
        if (r1 is None) != (r2 is None):
            raise ValueError("attn_paged: r1 and r2 come together")
        if out is None:
            out = torch.empty(T, H * dv, dtype=out_dtype, device=q.device)
        elif (out.dtype != out_dtype and out.dtype != torch.float32) or tuple(out.shape) != (T, H * dv):
            raise TypeError("attn_paged: out does not fit")
        _rows(out, "out")
        to = _code(out, "out")
        if head_gate is not None:
            _rows(head_gate, "head_gate", torch.float32)
            if tuple(head_gate.shape) != (T, H):
                raise ValueError("attn_paged: head_gate is [T, H]")
        if sink is not None and gate_bias is not None:
            raise ValueError("attn_paged: a silent softmax entry and per-key sigmoid weights exclude each other")
        extra = (1 if sink is not None else 0, float(sink or 0.0), head_gate.data_ptr() if head_gate is not None else None,
                 head_gate.stride(0) if head_gate is not None else 0)
        tiles = meta.get("q_tiles")
        if tiles is not None and kcache.dtype == torch.bfloat16 and d in (64, 128) and dv in (64, 128):
            # a step with many rows per request: the matrix-core kernel over row tiles
            rc = self.k.fls_seq_attn_prefill(q.data_ptr(), q.stride(0), _code(q, "q"), kcache.data_ptr(), ldk, vcache.data_ptr(),
                                             ldv, out.data_ptr(), to, out.stride(0), tiles.data_ptr(), tiles.shape[0],
                                             meta["tok_seq"].data_ptr(), meta["tok_pos"].data_ptr(), table.data_ptr(),
                                             table.stride(0), H, G, d, dv, float(scale), float(softcap),
                                             r1.data_ptr() if r1 is not None else None,
                                             r2.data_ptr() if r2 is not None else None, int(chunk), int(window),
                                             int(keep_first), gate_bias.data_ptr() if gate_bias is not None else None,
                                             float(out_scale), int(page_size), *extra, Gv, _stream())
            if rc == 0:
                return out
            if rc != -2:
                _chk(rc, "fls_seq_attn_prefill")
        bound = table.shape[1] * page_size                     # most keys a row can see
        if chunk > 0:
            bound = min(bound, int(chunk))
        if window > 0:
            bound = min(bound, int(window) + int(keep_first))
        if tiles is None and q.dtype == torch.float32 and kcache.dtype == torch.bfloat16 and gate_bias is None and r1 is None \
                and sink is None and head_gate is None and softcap == 0 and chunk == 0 and H // G <= 32 and Gv == G and to == 1 \
                and (d, dv) in self.HEAD_TILE_SHAPES:
            # few rows whose heads share long key / value rows (decoding over cached latent rows): the heads of a
            # token as the columns of one matrix-core tile, every key tile staged once for all of them
            ns = max(1, min(16, 256 // max(1, T * G), bound // 32))
            part = torch.empty(T * H * ns * (dv + 4), dtype=torch.float32, device=q.device) if ns > 1 else None
            rc = self.k.fls_seq_attn_heads(q.data_ptr(), q.stride(0), kcache.data_ptr(), ldk, vcache.data_ptr(), ldv,
                                           out.data_ptr(), out.stride(0), meta["tok_seq"].data_ptr(), meta["tok_pos"].data_ptr(),
                                           table.data_ptr(), table.stride(0), T, H, G, d, dv, float(scale), int(window),
                                           int(keep_first), float(out_scale), int(page_size), ns,
                                           part.data_ptr() if part is not None else None, _stream())
            if rc == 0:
                return out
            if rc != -2:
                _chk(rc, "fls_seq_attn_heads")
        # few rows over many keys (decoding a small batch): cut every row's keys into ranges that run as
        # blocks of their own, so that the launch has a few hundred blocks
        nsplit = max(1, min(8, 512 // max(1, T * H), bound // 256))
        part = torch.empty(T * H * nsplit * (dv + 4), dtype=torch.float32, device=q.device) if nsplit > 1 else None
        _chk(self.k.fls_seq_attn_paged(q.data_ptr(), q.stride(0), _code(q, "q"), kcache.data_ptr(), ldk, vcache.data_ptr(), ldv,
                                       _code(kcache, "kcache"), out.data_ptr(), to, out.stride(0), meta["tok_seq"].data_ptr(),
                                       meta["tok_pos"].data_ptr(), table.data_ptr(), table.stride(0), T, H, G, d, dv,
                                       float(scale), float(softcap), r1.data_ptr() if r1 is not None else None,
                                       r2.data_ptr() if r2 is not None else None, int(chunk), int(window), int(keep_first),
                                       gate_bias.data_ptr() if gate_bias is not None else None, float(out_scale),
                                       int(page_size), nsplit, part.data_ptr() if part is not None else None, *extra, Gv,
                                       _stream()), "fls_seq_attn_paged")
        return out

    # ------------------------------------------------------------ recurrences
    def causal_conv(self, x, w, b, state, meta, act="none", residual=False, out_dtype=torch.float32):
        _rows(x, "x", torch.float32)
        T, C = x.shape
        taps = w.shape[1]
        _vec(w, "w", C * taps)
        if b is not None:
            _vec(b, "b", C)
        if state.dtype != torch.float32 or not state.is_contiguous() or tuple(state.shape[1:]) != (taps - 1, C):
            raise ValueError("causal_conv: state must be fp32 [slots, taps - 1, C]")
        out = torch.empty(T, C, dtype=out_dtype, device=x.device)
        _chk(self.k.fls_seq_causal_conv(x.data_ptr(), x.stride(0), w.data_ptr(), b.data_ptr() if b is not None else None,
                                        state.data_ptr(), out.data_ptr(), _CODE[out_dtype], C, meta["tok_seq"].data_ptr(),
                                        meta["cu"].data_ptr(), meta["pos0"].data_ptr(), meta["slot"].data_ptr(), T,
                                        meta["n_seqs"], C, taps, 1 if act == "silu" else 0, 1 if residual else 0,
                                        1 if meta.get("max_rows") == 1 else 0, _stream()),
             "fls_seq_causal_conv")
        return out

    def delta_rule_scan(self, r, k, v, a, wz, g, w0, norm_w, state, meta, heads, dim, decay_scale, key_eps, norm_eps,
                        out_scale, out):
        T, hd = r.shape[0], heads * dim
        for nme, t in (("r", r), ("k", k), ("v", v), ("a", a), ("wz", wz), ("g", g)):
            _rows(t, nme, torch.float32)
            if tuple(t.shape) != (T, hd):
                raise ValueError(f"delta_rule_scan: {nme} is {tuple(t.shape)}, not {(T, hd)}")
        _rows(out, "out")
        _vec(w0, "w0", hd)
        _vec(norm_w, "norm_w", hd)
        if tuple(out.shape) != (T, hd) or tuple(state.shape[1:]) != (heads, dim, dim) or not state.is_contiguous() \
                or state.dtype != torch.float32:
            raise ValueError("delta_rule_scan: shapes do not fit")
        # a step with many rows per request and few (head, request) pairs: cut every state's columns over
        # 2 or 4 blocks so that the launch fills the chip
        splits = 1
        if meta.get("q_tiles") is not None:
            while heads * meta["n_seqs"] * splits < 512 and splits < 4 and dim % (2 * splits) == 0 and dim // (2 * splits) >= 8:
                splits *= 2
        raw = torch.empty(T * hd, dtype=torch.float32, device=r.device) if splits > 1 else None
        _chk(self.k.fls_seq_delta_rule_scan(r.data_ptr(), r.stride(0), k.data_ptr(), k.stride(0), v.data_ptr(), v.stride(0),
                                            a.data_ptr(), a.stride(0), wz.data_ptr(), wz.stride(0), g.data_ptr(), g.stride(0),
                                            w0.data_ptr(), norm_w.data_ptr(), state.data_ptr(), out.data_ptr(),
                                            _code(out, "out"), out.stride(0), meta["cu"].data_ptr(), meta["pos0"].data_ptr(),
                                            meta["slot"].data_ptr(), T, meta["n_seqs"], heads, dim, float(decay_scale),
                                            float(key_eps), float(norm_eps), float(out_scale), splits,
                                            raw.data_ptr() if raw is not None else None, _stream()),
             "fls_seq_delta_rule_scan")
        return out

    def rglru_scan(self, u, g, lam, y, state, meta, c, out_dtype):
        _rows(u, "u", torch.float32)
        _rows(g, "g", torch.float32)
        _rows(y, "y", torch.float32)
        T, Wd = u.shape
        if g.shape[1] != 2 * Wd or y.shape[1] != Wd or tuple(state.shape[1:]) != (Wd,) or not state.is_contiguous():
            raise ValueError("rglru_scan: shapes do not fit")
        _vec(lam, "lam", Wd)
        out = torch.empty(T, Wd, dtype=out_dtype, device=u.device)
        tiles, tile_cu = meta.get("q_tiles"), meta.get("tile_cu")
        if tiles is not None and tile_cu is not None:
            # many rows per request: three passes over row tiles instead of one thread per prompt and channel
            scratch = torch.empty(2 * tiles.shape[0] * Wd, dtype=torch.float32, device=u.device)
            _chk(self.k.fls_seq_rglru_scan_tiled(u.data_ptr(), u.stride(0), g.data_ptr(), g.stride(0), lam.data_ptr(),
                                                 y.data_ptr(), y.stride(0), state.data_ptr(), out.data_ptr(),
                                                 _CODE[out_dtype], Wd, tiles.data_ptr(), tiles.shape[0], tile_cu.data_ptr(),
                                                 scratch.data_ptr(), meta["pos0"].data_ptr(), meta["slot"].data_ptr(),
                                                 meta["n_seqs"], Wd, float(c), _stream()), "fls_seq_rglru_scan_tiled")
            return out
        _chk(self.k.fls_seq_rglru_scan(u.data_ptr(), u.stride(0), g.data_ptr(), g.stride(0), lam.data_ptr(), y.data_ptr(),
                                       y.stride(0), state.data_ptr(), out.data_ptr(), _CODE[out_dtype], Wd,
                                       meta["cu"].data_ptr(), meta["pos0"].data_ptr(), meta["slot"].data_ptr(),
                                       meta["n_seqs"], Wd, float(c), _stream()), "fls_seq_rglru_scan")
        return out

    def ssd_scan(self, xbc, z, dt, dt_bias, A_log, Dskip, state, meta, nh, P, N, G):
        _rows(xbc, "xbc", torch.float32)
        _rows(z, "z", torch.float32)
        _rows(dt, "dt", torch.float32)
        T, inner = xbc.shape[0], nh * P
        if xbc.shape[1] != inner + 2 * G * N or z.shape[1] != inner or dt.shape[1] != nh \
                or tuple(state.shape[1:]) != (nh, N, P) or not state.is_contiguous():
            raise ValueError("ssd_scan: shapes do not fit")
        for n, t in (("dt_bias", dt_bias), ("A_log", A_log), ("D", Dskip)):
            _vec(t, n, nh)
        out = torch.empty(T, inner, dtype=torch.float32, device=xbc.device)
        _chk(self.k.fls_seq_ssd_scan(xbc.data_ptr(), xbc.stride(0), z.data_ptr(), z.stride(0), dt.data_ptr(), dt.stride(0),
                                     dt_bias.data_ptr(), A_log.data_ptr(), Dskip.data_ptr(), state.data_ptr(),
                                     out.data_ptr(), inner, meta["cu"].data_ptr(), meta["pos0"].data_ptr(),
                                     meta["slot"].data_ptr(), meta["n_seqs"], nh, P, N, G, _stream()), "fls_seq_ssd_scan")
        return out

    # ------------------------------------------------------ mixture of experts
    def moe_route_topk(self, logits, top):
        """The ``top`` largest logits choose; the softmax over the chosen logits weighs."""
        return self.moe_route_corrected(logits, None, top)

    def moe_combine_(self, x, y, route, mult, shared=None, shared_gate=None):
        _rows(x, "x", torch.float32)
        _rows(y, "y", torch.float32)
        T, top = route.dest.shape
        D = x.shape[1]
        if x.shape[0] != T or y.shape[1] != D:
            raise ValueError("moe_combine_: shapes do not fit")
        if shared is not None:
            _rows(shared, "shared", torch.float32)
            if tuple(shared.shape) != (T, D):
                raise ValueError("moe_combine_: the shared expert's rows do not fit")
            if shared_gate is not None:
                _rows(shared_gate, "shared_gate", torch.float32)
                if tuple(shared_gate.shape) != (T, 1):
                    raise ValueError("moe_combine_: shared_gate is [T, 1]")
        _chk(self.k.fls_seq_moe_combine(x.data_ptr(), x.stride(0), y.data_ptr(), y.stride(0), route.dest.data_ptr(),
                                        route.w.data_ptr(), T, top, shared.data_ptr() if shared is not None else None,
                                        shared.stride(0) if shared is not None else 0,
                                        shared_gate.data_ptr() if shared is not None and shared_gate is not None else None,
                                        shared_gate.stride(0) if shared is not None and shared_gate is not None else 0, D,
                                        float(mult), _stream()), "fls_seq_moe_combine")
        return x

    def moe_route_corrected(self, logits, corr, top):
        """``corr`` None: top-k on the bare logits, softmax over the chosen."""
        _rows(logits, "logits", torch.float32)
        T, E = logits.shape
        if corr is not None:
            _vec(corr, "corr", E)
        dev = logits.device
        ids = torch.empty(T, top, dtype=torch.int32, device=dev)
        w = torch.empty(T, top, dtype=torch.float32, device=dev)
        ints = torch.zeros(3 * E + 1, dtype=torch.int32, device=dev)          # hist | cursor | offs
        hist, cursor, offs = ints[:E], ints[E:2 * E], ints[2 * E:]
        dest = torch.empty(T, top, dtype=torch.int32, device=dev)
        rows = torch.empty(T * top, dtype=torch.int32, device=dev)
        s = _stream()
        _chk(self.k.fls_seq_moe_route(logits.data_ptr(), logits.stride(0), corr.data_ptr() if corr is not None else None, T, E, top, ids.data_ptr(),
                                      w.data_ptr(), hist.data_ptr(), s), "fls_seq_moe_route")
        _chk(self.k.fls_seq_moe_scan(hist.data_ptr(), E, offs.data_ptr(), cursor.data_ptr(), s), "fls_seq_moe_scan")
        _chk(self.k.fls_seq_moe_place(ids.data_ptr(), T * top, top, cursor.data_ptr(), dest.data_ptr(), rows.data_ptr(), s),
             "fls_seq_moe_place")
        return SeqRoute(ids, w, offs, rows, dest, top)

    def moe_weighted_sum(self, y, route):
        _rows(y, "y", torch.float32)
        T, top = route.dest.shape
        out = torch.empty(T, y.shape[1], dtype=torch.float32, device=y.device)
        _chk(self.k.fls_seq_moe_sum(y.data_ptr(), y.stride(0), route.dest.data_ptr(), route.w.data_ptr(), out.data_ptr(),
                                    y.shape[1], T, top, y.shape[1], _stream()), "fls_seq_moe_sum")
        return out
