"""Each kernel of ``csrc/kernels/seq`` against the plain PyTorch op of the same name
(``ops/torch_seq.py``, fp32 arithmetic), on shapes that exercise every tile path, tail and batch form:
GEMMs (64 / 128 / 256 tiles, the skinny decode kernel, K tails, column-slice operands, strided batch,
row groups), group norm, activations, K/V store, both attention kernels over paged keys (chunks, windows,
carried positions, head sizes on and off the matrix-core path), convolution and both scans with carried
state in scattered slots, routing."""
import numpy as np
import pytest
import torch

from conftest import gpu_available

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    if not gpu_available():
        pytest.skip("no GPU")
    from flexible_llm_sharding_amd.ops.hip_seq import HipSeqOps
    from flexible_llm_sharding_amd.ops.torch_seq import TorchSeqOps
    return HipSeqOps(), TorchSeqOps()


def close(a, b, tol):
    a, b = a.float().cpu(), b.float().cpu()
    e = (a - b).abs().max().item() / (b.abs().max().item() + 1e-9)
    assert e < tol, e


def meta_of(lens, pos0, dev, ps=16, seed=0):
    rng = np.random.default_rng(seed)
    B = len(lens)
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    seq = np.repeat(np.arange(B), lens).astype(np.int32)
    pos = np.concatenate([np.arange(p, p + n) for p, n in zip(pos0, lens)]).astype(np.int32)
    npg = [-(-(p + n) // ps) for p, n in zip(pos0, lens)]
    tab = np.full((B, max(npg)), -1, np.int32)
    perm = rng.permutation(sum(npg) + 5)
    k = 0
    for b in range(B):
        for j in range(npg[b]):
            tab[b, j] = perm[k]
            k += 1
    slot = rng.permutation(B + 3)[:B].astype(np.int32)
    kvs = (tab[seq, pos // ps].astype(np.int64) * ps + pos % ps).astype(np.int32)
    m = dict(tok_seq=seq, tok_pos=pos, cu=cu, pos0=np.array(pos0, np.int32), slot=slot, page_table=tab, kv_slot=kvs)
    md = {k: torch.from_numpy(v).to(dev) for k, v in m.items()}
    md.update(n_seqs=B, cu_host=cu, pos0_host=np.array(pos0), max_rows=max(lens))
    if max(lens) >= 16:
        md["q_tiles"] = torch.tensor([(a + o, min(128, b - a - o)) for a, b in zip(cu[:-1], cu[1:])
                                      for o in range(0, b - a, 128)], dtype=torch.int32, device=dev)
        md["tile_cu"] = torch.tensor(np.concatenate([[0], np.cumsum([-(-int(n) // 128) for n in lens])]), dtype=torch.int32,
                                     device=dev)
    return md, sum(npg) + 5, B + 3


DTYPES = [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)]
DEV = "cuda:0"


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("M,N,K", [(5, 70, 33), (130, 192, 256), (64, 64, 64), (1, 454, 256), (300, 200, 454), (257, 129, 72),
                                   (4100, 4200, 136), (8, 200, 512), (32, 64, 72), (17, 100, 2056), (3, 4096, 1024)])
def test_matmul(ops, cdt, tol, M, N, K):
    H, R = ops
    torch.manual_seed(M + N + K)
    a = torch.randn(M, K, device=DEV).to(cdt)
    w = torch.randn(N, K, device=DEV).to(cdt)
    b = torch.randn(N, device=DEV)
    close(H.matmul_nt(a, w, b), R.matmul_nt(a, w, b), 1e-5)
    act = torch.tensor([0.4, -0.3], device=DEV)                     # activation and rounding in the epilogue
    close(H.matmul_nt(a, w, b, xielu=act, out_dtype=cdt), R.matmul_nt(a, w, b, xielu=act, out_dtype=cdt), tol)
    af = torch.randn(M, K + 8, device=DEV)[:, 4:4 + K]             # fp32 rows, a column slice: rounded on the way in
    close(H.matmul_nt(af, w), R.matmul_nt(af.to(cdt), w), 1e-5)


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_rows(ops, cdt, tol):
    H, R = ops
    torch.manual_seed(1)
    x = torch.randn(37, 96, device=DEV)
    w = torch.randn(96, device=DEV)
    idx = torch.tensor([3, 0, 36, 5], dtype=torch.int32, device=DEV)
    close(H.group_rmsnorm(x, w, 3, 1e-6, cdt), R.group_rmsnorm(x, w, 3, 1e-6, cdt), tol)
    close(H.group_rmsnorm(x, w, 1, 1e-6, cdt, row_idx=idx), R.group_rmsnorm(x, w, 1, 1e-6, cdt, row_idx=idx), tol)
    x1, x2, y = x.clone(), x.clone(), torch.randn(37, 96, device=DEV)
    close(H.add_group_rmsnorm_(x1, y, w, 2, 1e-6), R.add_group_rmsnorm_(x2, y, w, 2, 1e-6), 1e-5)
    u = torch.randn(9, 48, device=DEV)
    wg = torch.randn(6, 16, 16, device=DEV).to(cdt)
    bg = torch.randn(96, device=DEV)
    close(H.block_linear(u, wg, bg, 3, cdt), R.block_linear(u, wg, bg, 3, cdt), 1e-5)
    z = torch.randn(11, 50, device=DEV) * 3
    act = torch.tensor([0.3, -0.2], device=DEV)
    close(H.xielu(z, act, cdt), R.xielu(z, act, cdt), tol)
    close(H.silu_mul(z, cdt), R.silu_mul(z, cdt), tol)
    close(H.softcap_(z.clone(), 5.0), R.softcap_(z.clone(), 5.0), 1e-5)
    assert bool((H.argmax_f32(z).cpu() == R.argmax_f32(z).cpu()).all())
    tab = torch.randn(40, 24, device=DEV).to(cdt)
    ids = torch.tensor([1, 39, 0, 7], dtype=torch.int32, device=DEV)
    close(H.embed_rows(ids, tab), R.embed_rows(ids, tab), 1e-6)


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("Hh,G,d,dv", [(6, 2, 24, 40), (6, 2, 64, 64), (4, 4, 128, 64), (8, 2, 128, 128), (2, 1, 64, 128)])
def test_attention(ops, cdt, tol, Hh, G, d, dv):
    H, R = ops
    torch.manual_seed(d + dv)
    for lens, pos0, chunk, window in (([70, 5, 33], [0, 0, 0], 20, 0), ([3, 1, 1], [70, 5, 33], 20, 0), ([40, 17], [0, 0], 0, 9),
                                      ([2, 2], [40, 17], 0, 9), ([150], [0], 64, 0), ([300, 17, 140], [0, 0, 0], 100, 0),
                                      ([200, 30], [300, 17], 100, 0), ([260], [0], 0, 50), ([260], [0], 0, 0)):
        md, npages, _ = meta_of(lens, pos0, DEV)
        T = sum(lens)
        kc = torch.randn(npages, 16, G * d, device=DEV).to(cdt)
        vc = torch.randn(npages, 16, G * dv, device=DEV).to(cdt)
        kc2, vc2 = kc.clone(), vc.clone()
        k, v, kn = torch.randn(T, G * d, device=DEV), torch.randn(T, G * dv, device=DEV), torch.randn(G * d, device=DEV)
        H.kv_store(k, kn, 1e-6, v, kc, vc, md["kv_slot"])
        R.kv_store(k, kn, 1e-6, v, kc2, vc2, md["kv_slot"])
        close(kc, kc2, tol)
        close(vc, vc2, tol)
        q = torch.randn(T, Hh * d, device=DEV).to(cdt)
        r1, r2 = torch.rand(Hh, device=DEV), torch.rand(Hh, device=DEV)
        o1 = H.attn_paged(q, kc2, vc2, md, Hh, G, d, dv, 0.3, 8.0, r1, r2, chunk, 16, cdt, window=window)
        o2 = R.attn_paged(q, kc2, vc2, md, Hh, G, d, dv, 0.3, 8.0, r1, r2, chunk, 16, cdt, window=window)
        close(o1, o2, tol)


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_conv_and_scans_carry_state(ops, cdt, tol):
    H, R = ops
    torch.manual_seed(3)
    for lens, pos0 in (([9, 1, 4], [0, 0, 0]), ([2, 1, 1], [9, 1, 4]), ([1, 1, 1], [11, 2, 5]), ([40, 3], [0, 7]), ([300, 5, 129], [0, 0, 6])):
        md, _, nslots = meta_of(lens, pos0, DEV)
        T, C, taps = sum(lens), 70, 4
        x = torch.randn(T, C + 6, device=DEV)[:, 3:3 + C]
        w, b = torch.randn(C, taps, device=DEV), torch.randn(C, device=DEV)
        st = torch.randn(nslots, taps - 1, C, device=DEV)
        st2 = st.clone()
        close(H.causal_conv(x, w, b, st, md, "silu"), R.causal_conv(x, w, b, st2, md, "silu"), 1e-5)
        close(st, st2, 1e-6)
        Wd = 70
        u, g = torch.randn(T, Wd, device=DEV), torch.randn(T, 2 * Wd, device=DEV)
        lam, y = torch.randn(Wd, device=DEV), torch.randn(T, Wd, device=DEV)
        s1 = torch.randn(nslots, Wd, device=DEV)
        s2 = s1.clone()
        close(H.rglru_scan(u, g, lam, y, s1, md, 8.0, cdt), R.rglru_scan(u, g, lam, y, s2, md, 8.0, cdt), tol)
        close(s1, s2, 1e-5)
        for nh, P, N, Gg in ((6, 20, 24, 2), (4, 64, 128, 1), (3, 8, 16, 3), (2, 40, 200, 1)):
            inner = nh * P
            xbc = torch.randn(T, inner + 2 * Gg * N, device=DEV)
            zz, dt = torch.randn(T, inner, device=DEV), torch.randn(T, nh, device=DEV)
            dtb, Al, Ds = torch.randn(nh, device=DEV), torch.randn(nh, device=DEV) * 0.5, torch.randn(nh, device=DEV)
            s1 = torch.randn(nslots, nh, N, P, device=DEV)
            s2 = s1.clone()
            close(H.ssd_scan(xbc, zz, dt, dtb, Al, Ds, s1, md, nh, P, N, Gg), R.ssd_scan(xbc, zz, dt, dtb, Al, Ds, s2, md, nh, P, N, Gg), 3e-5)
            close(s1, s2, 3e-5)


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("T,E,top", [(33, 10, 3), (700, 8, 2), (5, 40, 9), (300, 3, 1), (4, 8, 2), (10, 6, 3), (1, 5, 5)])
def test_routing_and_expert_products(ops, cdt, tol, T, E, top):
    H, R = ops
    torch.manual_seed(T)
    D, ff = 48, 20
    lg, corr = torch.randn(T, E, device=DEV), torch.randn(E, device=DEV) * 0.1
    a, b = H.moe_route_corrected(lg, corr, top), R.moe_route_corrected(lg, corr, top)
    assert bool((a.ids.cpu() == b.ids.cpu()).all()) and bool((a.offs.cpu() == b.offs.cpu()).all())
    # every sorted row sits in its expert's range and maps back to its token
    offs, rows, dest = a.offs.cpu().numpy(), a.rows.cpu().numpy(), a.dest.cpu().numpy()
    ids = a.ids.cpu().numpy()
    assert sorted(dest.reshape(-1).tolist()) == list(range(T * top))
    for t in range(T):
        for k in range(top):
            assert offs[ids[t, k]] <= dest[t, k] < offs[ids[t, k] + 1] and rows[dest[t, k]] == t
    close(a.w, b.w, 1e-5)
    h = torch.randn(T, D, device=DEV).to(cdt)
    wgu = torch.randn(E, 2 * ff, D, device=DEV).to(cdt)
    o1 = H.moe_weighted_sum(H.grouped_matmul_nt(H.gather_rows(h, a.rows), wgu, a.offs), a)
    o2 = R.moe_weighted_sum(R.grouped_matmul_nt(R.gather_rows(h, b.rows), wgu, b.offs), b)
    close(o1, o2, 1e-5)


# ------------------------------------------------ kernels of the latent / gated-attention / delta-rule mixers
@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_norm_offset_gate_unary_and_head_products(ops, cdt, tol):
    H, R = ops
    torch.manual_seed(3)
    x = torch.randn(37, 90, device=DEV)
    w = torch.randn(90, device=DEV) * 0.3
    close(H.group_rmsnorm(x, w, 1, 1e-5, cdt, w_offset=1.0), R.group_rmsnorm(x, w, 1, 1e-5, cdt, w_offset=1.0), tol)
    y1, y2 = torch.randn(37, 90, device=DEV), None
    a, b = x.clone(), x.clone()
    close(H.add_group_rmsnorm_(a, y1, w, 3, 1e-5, w_offset=1.0), R.add_group_rmsnorm_(b, y1, w, 3, 1e-5, w_offset=1.0), 2e-6)
    gu = torch.randn(37, 2 * 70, device=DEV) * 2
    for act in ("silu", "gelu_tanh"):
        close(H.gate_mul(gu, cdt, act), R.gate_mul(gu, cdt, act), tol)
    close(H.unary(gu[:, 3:50], "tanh", cdt), R.unary(gu[:, 3:50], "tanh", cdt), tol)
    # per-head products: heads read strided column blocks of a and write strided column blocks of out
    for T in (1, 5, 200):
        heads, K, N, a_hs, o_hs = 5, 24, 13, 30, 20
        av = torch.randn(T, heads * a_hs, device=DEV)
        wv = torch.randn(heads, N, K, device=DEV).to(cdt)
        o1 = torch.full((T, heads * o_hs), 7.0, device=DEV)
        o2 = o1.clone()
        H.head_matmul_nt(av, wv, heads, a_hs, o1, o_hs)
        R.head_matmul_nt(av, wv, heads, a_hs, o2, o_hs)
        close(o1, o2, tol)
        assert (o1[:, N:o_hs] == 7.0).all()               # columns between the heads' blocks stay untouched


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_head_norm_rope(ops, cdt, tol):
    H, R = ops
    torch.manual_seed(4)
    lens, pos0 = [1, 40, 3, 130], [900, 0, 17, 5000]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    T = sum(lens)
    for heads, n, x_col, x_hs, rot, with_w in ((3, 24, 5, 30, 10, True), (1, 14, 0, 0, 0, True), (1, 6, 14, 0, 6, False),
                                               (2, 200, 8, 200, 64, True), (4, 64, 0, 64, 64, True)):
        x = torch.randn(T, x_col + heads * max(x_hs, n) + 3, device=DEV)
        w = torch.randn(n, device=DEV) if with_w else None
        o_hs, o_col = n + 4, 2
        for paged in (False, True):
            rows = n_pages * 16 if paged else T
            outs = []
            for O in (H, R):
                out = torch.zeros(rows, o_col + heads * o_hs, device=DEV, dtype=cdt)
                raw = torch.zeros_like(out)
                O.head_norm_rope(x, heads, n, x_col, x_hs, out, o_col, o_hs, md, w=w, eps=1e-5,
                                 rot=(rot, 5000.0) if rot else None, row_map=md["kv_slot"] if paged else None, raw=raw)
                outs.append((out, raw))
            close(outs[0][0], outs[1][0], max(tol, 3e-4))     # (angles of thousands of radians in fp32)
            close(outs[0][1], outs[1][1], tol)


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("Hh,G,d,dv,ldk,ldv,shared", [(6, 2, 24, 24, 48, 48, False), (3, 1, 20, 14, 20, 20, True),
                                                      (5, 1, 72, 56, 72, 72, True), (4, 4, 64, 64, 256, 256, False)])
def test_attention_windows_kept_tokens_and_gates(ops, cdt, tol, Hh, G, d, dv, ldk, ldv, shared):
    H, R = ops
    torch.manual_seed(5)
    lens, pos0 = [1, 70, 2, 33, 1], [150, 0, 64, 31, 3]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    T = sum(lens)
    kc = (torch.randn(n_pages, 16, ldk, device=DEV) * 0.5).to(cdt)
    vc = kc if shared else (torch.randn(n_pages, 16, ldv, device=DEV)).to(cdt)
    gb = torch.randn(Hh, device=DEV)
    for q_dt in (torch.float32, cdt):
        q = torch.randn(T, Hh * d, device=DEV).to(q_dt)
        for window, keep, gate, scale_out in ((9, 0, None, 1.0), (9, 4, None, 0.6), (40, 20, gb, 1.0), (1, 0, gb, 1.7), (40, 3, gb, 0.5),
                                              (1000, 0, None, 1.0)):
            kw = dict(scale=0.2, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=window,
                      keep_first=keep, gate_bias=gate, out_scale=scale_out)
            a = H.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw)
            b = R.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw)
            close(a, b, tol)
    # into a column block of a wider matrix
    q = torch.randn(T, Hh * d, device=DEV)
    wide = torch.zeros(T, Hh * dv + 10, device=DEV, dtype=cdt)
    kw = dict(scale=0.2, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=9, keep_first=2, gate_bias=gb)
    H.attn_paged(q, kc, vc, md, Hh, G, d, dv, out=wide[:, :Hh * dv], **kw)
    close(wide[:, :Hh * dv], R.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), tol)
    assert (wide[:, Hh * dv:] == 0).all()


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("heads,dim", [(3, 7), (2, 32), (1, 33), (4, 64), (2, 100), (3, 128), (5, 1)])
def test_input_conv_and_delta_rule_carry_state(ops, cdt, tol, heads, dim):
    H, R = ops
    torch.manual_seed(6 + dim)
    hd = heads * dim
    state = None
    for step, (lens, pos0) in enumerate((([40, 1, 3, 150], [0, 0, 0, 0]), ([1, 1, 1, 1], [40, 1, 3, 150]), ([2, 17, 1, 30], [41, 2, 4, 151]))):
        md, _, n_slots = meta_of(lens, pos0, DEV, seed=1)          # (the same slots in every step)
        T = sum(lens)
        # the input convolution: residual form, no bias, output of the GEMM type
        C = 50
        x = torch.randn(T, C, device=DEV)
        if step == 0:
            cs1 = {taps: torch.randn(n_slots, taps - 1, C, device=DEV) for taps in (1, 2, 4, 9)}
            cs2 = {taps: t.clone() for taps, t in cs1.items()}
            s1 = torch.randn(n_slots, heads, dim, dim, device=DEV)
            s2 = s1.clone()
        for taps in (1, 2, 4, 9):                                  # (nine taps: the kernel without the register window)
            cw = torch.randn(C, taps, device=DEV) * 0.5
            close(H.causal_conv(x, cw, None, cs1[taps], md, residual=True, out_dtype=cdt),
                  R.causal_conv(x, cw, None, cs2[taps], md, residual=True, out_dtype=cdt), tol)
            if taps > 1:
                close(cs1[taps][md["slot"].long()], cs2[taps][md["slot"].long()], 1e-6)
        z = torch.randn(T, 6 * hd + 5, device=DEV)
        r, k, v, a, wz, g = (z[:, i * hd:(i + 1) * hd] for i in range(6))
        w0, nw = torch.randn(hd, device=DEV) - 2.0, torch.randn(hd, device=DEV)
        o1 = torch.zeros(T, hd + 3, device=DEV, dtype=cdt)
        o2 = torch.zeros_like(o1)
        kw = dict(decay_scale=0.6065, key_eps=1e-6, norm_eps=1e-5, out_scale=1.3)
        H.delta_rule_scan(r, k, v, a, wz, g, w0, nw, s1, md, heads, dim, out=o1[:, :hd], **kw)
        R.delta_rule_scan(r, k, v, a, wz, g, w0, nw, s2, md, heads, dim, out=o2[:, :hd], **kw)
        close(o1, o2, max(tol, 2e-4))
        close(s1[md["slot"].long()], s2[md["slot"].long()], 2e-4)


@pytest.mark.parametrize("d,dv", [(64, 64), (128, 128), (128, 64)])
def test_matrix_core_attention_over_row_tiles(ops, d, dv):
    """bf16 prompts of several 128-row tiles through the matrix-core kernel (fp32 and bf16 queries):
    windows shorter and longer than a tile, kept first keys filling more than one key tile, sigmoid
    gates, pool rows wider than the heads, and a step-local table of one-row pages."""
    H, R = ops
    torch.manual_seed(8)
    cdt = torch.bfloat16
    Hh, G = 4, 2
    lens, pos0 = [300, 17, 129], [0, 0, 0]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    T = sum(lens)
    kc = (torch.randn(n_pages, 16, G * d + 16, device=DEV) * 0.5).to(cdt)
    vc = torch.randn(n_pages, 16, G * dv + 8, device=DEV).to(cdt)
    gb = torch.randn(Hh, device=DEV)
    for q_dt in (torch.float32, cdt):
        q = torch.randn(T, Hh * d, device=DEV).to(q_dt)
        for window, keep, gate in ((40, 0, None), (40, 50, None), (200, 70, gb), (7, 3, gb), (1000, 0, gb)):
            kw = dict(scale=d ** -0.5, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=window,
                      keep_first=keep, gate_bias=gate, out_scale=0.8)
            close(H.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), R.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), 2e-2)
    # keys and values of the step itself, one row a page, every head its own
    cu = md["cu_host"]
    local = torch.from_numpy((cu[:-1, None] + np.arange(max(lens))[None, :]).astype(np.int32)).to(DEV)
    kf = (torch.randn(T, 1, Hh * d, device=DEV) * 0.5).to(cdt)
    vf = torch.randn(T, 1, Hh * dv, device=DEV).to(cdt)
    q = torch.randn(T, Hh * d, device=DEV)
    kw = dict(scale=d ** -0.5, softcap=0.0, r1=None, r2=None, chunk=0, page_size=1, out_dtype=cdt, window=33)
    lm = dict(md, page_table=local)
    close(H.attn_paged(q, kf, vf, lm, Hh, Hh, d, dv, **kw), R.attn_paged(q, kf, vf, lm, Hh, Hh, d, dv, **kw), 2e-2)


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_decode_rows_over_long_contexts_split_their_keys(ops, cdt, tol):
    """Three decode rows far into their sequences: the launch cuts every row's keys into ranges that run
    as blocks of their own and merges them (softmax parts by their maxima and sums, gated parts by
    addition); a row near the start has ranges without keys."""
    H, R = ops
    torch.manual_seed(9)
    lens, pos0 = [1, 1, 1], [1500, 3, 700]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    Hh, G, d, dv = 4, 2, 24, 40
    kc = (torch.randn(n_pages, 16, G * d, device=DEV) * 0.5).to(cdt)
    vc = torch.randn(n_pages, 16, G * dv, device=DEV).to(cdt)
    q = torch.randn(3, Hh * d, device=DEV)
    gb = torch.randn(Hh, device=DEV)
    for window, keep, gate in ((0, 0, None), (1000, 0, None), (600, 90, gb), (0, 0, gb)):
        kw = dict(scale=0.3, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=window,
                  keep_first=keep, gate_bias=gate, out_scale=0.9)
        close(H.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), R.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), tol)


@pytest.mark.parametrize("d,dv,Hh", [(192, 128, 5), (320, 256, 32), (576, 512, 16)])
def test_heads_of_a_token_share_one_matrix_core_tile(ops, d, dv, Hh):
    """Decode rows over latent rows (one key / value head, values = the first columns of the key rows):
    the kernel that takes a token's heads as the columns of one tile, with the keys cut over several
    blocks and merged, rows with fewer keys than a tile, windows and kept first keys."""
    H, R = ops
    torch.manual_seed(10)
    cdt = torch.bfloat16
    lens, pos0 = [1, 1, 1, 1], [1500, 3, 700, 31]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    pool = (torch.randn(n_pages, 16, d, device=DEV) * 0.3).to(cdt)
    q = torch.randn(4, Hh * d, device=DEV)
    for window, keep in ((0, 0), (1000, 0), (600, 90), (33, 0)):
        kw = dict(scale=d ** -0.5, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=window,
                  keep_first=keep, out_scale=0.9)
        close(H.attn_paged(q, pool, pool, md, Hh, 1, d, dv, **kw), R.attn_paged(q, pool, pool, md, Hh, 1, d, dv, **kw), 2e-2)


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_dyt_norm_scaled_add_and_embedding_scale(ops, cdt, tol):
    """Dynamic Tanh norm (vector path and odd widths, row gather, column slices), x += m y, embedding rows times a scale."""
    H, R = ops
    torch.manual_seed(11)
    for T, D in ((7, 320), (3, 37), (130, 2048), (1, 4100)):
        x = torch.randn(T, D + 8, device=DEV)[:, 4:4 + D] * 2
        wb = torch.randn(2, D, device=DEV)
        alpha = torch.tensor([0.7], device=DEV)
        close(H.dyt_norm(x, wb, alpha, cdt), R.dyt_norm(x, wb, alpha, cdt), tol)
        xc = x.contiguous()
        close(H.dyt_norm(xc, wb, alpha, cdt), R.dyt_norm(xc, wb, alpha, cdt), tol)
        idx = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32, device=DEV)
        close(H.dyt_norm(xc, wb, alpha, torch.float32, row_idx=idx), R.dyt_norm(xc, wb, alpha, torch.float32, row_idx=idx), 1e-5)
        y = torch.randn(T, D, device=DEV)
        a, b = xc.clone(), xc.clone()
        close(H.add_scaled_(a, y, 0.6), R.add_scaled_(b, y, 0.6), 1e-6)
        ys = torch.randn(T, D + 3, device=DEV)[:, 1:1 + D]
        close(H.add_scaled_(a, ys, -1.3), R.add_scaled_(b, ys, -1.3), 1e-6)
    table = torch.randn(50, 36, device=DEV).to(cdt)
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=DEV)
    close(H.embed_rows(ids, table, scale=0.37), R.embed_rows(ids, table, scale=0.37), 1e-6)


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_rotation_with_rescaled_frequencies_then_unit_norm(ops, cdt, tol):
    """Pair rotation with wavelength-rescaled frequencies followed by the weightless RMS norm, into rows and into pools;
    a plain placement (no norm, no rotation) of value heads."""
    H, R = ops
    torch.manual_seed(12)
    lens, pos0 = [1, 40, 3, 130], [900, 0, 17, 2000]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    T = sum(lens)
    sc = (8.0, 1.0, 4.0, 64)
    f = R.rope_freqs(16, 100.0, "cpu", sc).double()
    f0 = R.rope_freqs(16, 100.0, "cpu").double()
    ratio = (f / f0).numpy()
    assert ratio[0] == 1.0 and abs(ratio[-1] - 1 / 8) < 1e-6 and ((ratio[1:] <= ratio[:-1] + 1e-9).all())   # kept, blended, slowed
    assert ((ratio > 1 / 8 + 1e-3) & (ratio < 1 - 1e-3)).any()
    for heads, n, x_col, rot in ((3, 24, 5, (16, 100.0, sc)), (2, 40, 0, (40, 30000.0, (4.0, 2.0, 8.0, 512))), (4, 64, 0, (32, 1e4, None)),
                                 (1, 6, 2, None), (2, 130, 0, (128, 500.0, None))):
        x = torch.randn(T, x_col + heads * n + 3, device=DEV) * 3
        for paged in (False, True):
            rows = n_pages * 16 if paged else T
            outs = []
            for O in (H, R):
                out = torch.zeros(rows, heads * n, device=DEV, dtype=cdt)
                O.head_norm_rope(x, heads, n, x_col, n, out, 0, n, md, eps=1e-5, rot=rot, unit_after=True,
                                 row_map=md["kv_slot"] if paged else None)
                outs.append(out)
            close(outs[0], outs[1], max(tol, 3e-4))
            if not paged:                                       # every head has unit mean square
                ms = outs[0].float().view(T, heads, n).pow(2).mean(-1)
                assert (ms - 1).abs().max().item() < (2e-2 if cdt == torch.bfloat16 else 1e-3)


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("Hh,G,d,dv", [(5, 5, 40, 72), (6, 2, 24, 40), (4, 2, 64, 64), (8, 2, 128, 128), (4, 4, 128, 64), (3, 1, 20, 14)])
def test_attention_with_a_silent_softmax_entry_and_head_gates(ops, cdt, tol, Hh, G, d, dv):
    """Windowed softmax with one more entry of a given score and no value, and a sigmoid gate per (row, head): prompts
    (per-row kernel, and row tiles on the matrix cores where the head sizes allow), portions, decode rows."""
    H, R = ops
    torch.manual_seed(13)
    lens, pos0 = [1, 170, 2, 33, 1], [150, 0, 64, 31, 3]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    T = sum(lens)
    kc = (torch.randn(n_pages, 16, G * d, device=DEV) * 0.5).to(cdt)
    vc = torch.randn(n_pages, 16, G * dv, device=DEV).to(cdt)
    z = torch.randn(T, Hh * d + Hh + 5, device=DEV)
    hg = z[:, Hh * d:Hh * d + Hh]                               # a column block of a wider matrix
    q = torch.randn(T, Hh * d, device=DEV) * (8 / d) ** 0.5      # (scores of a few units whatever the head size)
    for window, sink, gate, scale in ((9, 0.0, hg, 0.2), (72, 0.0, hg, 0.5), (72, 1.5, None, 0.2), (1, 0.0, hg, 0.3), (0, -2.0, hg, 0.05),
                                      (40, None, hg, 0.2), (40, 0.0, hg, 1.5), (40, 0.0, hg, -1.5)):
        kw = dict(scale=scale, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=window, sink=sink,
                  head_gate=gate)
        a = H.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw)
        b = R.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw)
        close(a, b, tol)
    # decode rows far into their sequences: every row's keys cut over blocks, the silent entry joins once in the merge
    lens, pos0 = [1, 1, 1], [1500, 3, 700]
    md, n_pages, _ = meta_of(lens, pos0, DEV)
    kc = (torch.randn(n_pages, 16, G * d, device=DEV) * 0.5).to(cdt)
    vc = torch.randn(n_pages, 16, G * dv, device=DEV).to(cdt)
    q = torch.randn(3, Hh * d, device=DEV) * (8 / d) ** 0.5
    hg = torch.randn(3, Hh, device=DEV)
    for window, sink, scale in ((0, 0.0, 0.3), (1000, 0.0, 0.01), (1000, 3.0, 0.3), (600, 0.0, -1.0)):
        kw = dict(scale=scale, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, window=window, sink=sink, head_gate=hg)
        close(H.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), R.attn_paged(q, kc, vc, md, Hh, G, d, dv, **kw), tol)


@pytest.mark.parametrize("T,E,top", [(33, 10, 3), (700, 8, 2), (5, 40, 9), (300, 3, 1), (4, 8, 8), (1, 5, 5)])
def test_topk_routing_and_combine(ops, T, E, top):
    """The largest logits choose, the softmax over the chosen weighs; the combine adds the weighted expert rows, the gated
    shared expert's row and the residual in one pass."""
    H, R = ops
    torch.manual_seed(14)
    D = 52
    z = torch.randn(T, E + 3, device=DEV)
    logits = z[:, 1:1 + E]
    a, b = H.moe_route_topk(logits, top), R.moe_route_topk(logits, top)
    assert torch.equal(a.ids.cpu().long(), b.ids.cpu().long())
    close(a.w, b.w, 1e-5)
    assert (a.w.sum(-1) - 1).abs().max().item() < 1e-5
    assert torch.equal(a.offs.cpu().long(), b.offs.cpu().long())
    # a tie goes to the lower expert
    tie = torch.zeros(2, E, device=DEV)
    assert H.moe_route_topk(tie, top).ids.cpu().tolist() == [list(range(top))] * 2
    y = torch.randn(T * top, D, device=DEV)
    shared = torch.randn(T, D, device=DEV)
    gate = torch.randn(T, 4, device=DEV)[:, 2:3]
    for sh, g in ((None, None), (shared, gate), (shared, None)):
        x1, x2 = torch.randn(T, D, device=DEV), None
        x2 = x1.clone()
        H.moe_combine_(x1, y, a, 0.6, sh, g)
        R.moe_combine_(x2, y, a, 0.6, sh, g)
        close(x1, x2, 1e-5)


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("Hh,G,d,dv,taps,rot", [(6, 2, 24, 40, 3, (16, 100.0, (8.0, 1.0, 4.0, 64))), (3, 3, 40, 72, 4, (40, 3e4, None)),
                                                (4, 0, 64, 64, 2, (32, 1e4, None)), (2, 1, 128, 96, 1, (128, 5e5, None)),
                                                (2, 2, 10, 6, 10, None), (5, 1, 130, 200, 5, (64, 1e3, None))])
def test_projected_rows_into_attention_in_one_pass(ops, cdt, tol, Hh, G, d, dv, taps, rot):
    """Convolution with carried history, rotation, unit norm and page write of q | k | v rows as one kernel against the
    chain of plain ops: prompts, portions that continue a request, single decoded rows (which also rewrite the history),
    query-only layers (G = 0), one tap, no convolution at all."""
    H, R = ops
    torch.manual_seed(15)
    C = Hh * d + G * (d + dv)
    for lens, pos0 in (([1, 40, 3, 130], [900, 0, 17, 2000]), ([1, 1, 1], [5, 0, 300])):
        md, n_pages, n_slots = meta_of(lens, pos0, DEV)
        T = sum(lens)
        z = torch.randn(T, C + Hh + 3, device=DEV)
        for w in ((torch.randn(C, taps, device=DEV) * 0.5), None):
            st0 = torch.randn(n_slots, taps - 1, C, device=DEV) if (w is not None and taps > 1) else None
            outs = []
            for O in (H, R):
                st = st0.clone() if st0 is not None else None
                q = torch.zeros(T, Hh * d, device=DEV)
                kc = torch.zeros(n_pages, 16, max(G, 1) * d, device=DEV, dtype=cdt)
                vc = torch.zeros(n_pages, 16, max(G, 1) * dv, device=DEV, dtype=cdt)
                O.qkv_conv_rope_store(z, w, st, md, Hh, G, d, dv, q, kc if G else None, vc if G else None, eps=1e-5, rot=rot)
                outs.append((q, kc, vc, st))
            close(outs[0][0], outs[1][0], 3e-4)
            close(outs[0][1], outs[1][1], max(tol, 3e-4))
            close(outs[0][2], outs[1][2], tol) if G else None
            if st0 is not None:
                used = md["slot"].long()
                close(outs[0][3][used], outs[1][3][used], 1e-6)
                free = [i for i in range(n_slots) if i not in used.tolist()]
                assert torch.equal(outs[0][3][free], st0[free])


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_residual_add_with_the_next_norm(ops, cdt, tol):
    H, R = ops
    torch.manual_seed(16)
    for T, D in ((7, 320), (3, 37), (130, 2048)):
        x = torch.randn(T, D, device=DEV) * 2
        y = torch.randn(T, D + 4, device=DEV)[:, 2:2 + D]
        wb, alpha = torch.randn(2, D, device=DEV), torch.tensor([0.6], device=DEV)
        a, b = x.clone(), x.clone()
        ha, hb = H.add_scaled_dyt_norm_(a, y, 0.6, wb, alpha, cdt), R.add_scaled_dyt_norm_(b, y, 0.6, wb, alpha, cdt)
        close(a, b, 1e-6)
        close(ha, hb, tol)


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("S,D", [(1, 36), (3, 320), (5, 34), (2, 2304)])
def test_residual_streams_norm_update_and_embedding_copies(ops, cdt, tol, S, D):
    """Several residual streams side by side in a row: their weighted sum through the RMS norm (also the plain
    sum with a row gather), the update of all streams at once with the gated sublayer output (gate logits as a
    column block of a wider matrix), the same fused with the next norm, one stream without coefficients, and the
    embedding with a position vector written S times."""
    H, R = ops
    torch.manual_seed(S * D)
    T = 37
    xs = torch.randn(T, S * D, device=DEV)
    hc = torch.randn(2 * S + S * S, device=DEV)
    w = 1 + 0.3 * torch.randn(D, device=DEV)
    idx = torch.tensor([5, 0, 36, 5], dtype=torch.int32, device=DEV)
    close(H.streams_norm(xs, hc, w, 1e-5, cdt, S), R.streams_norm(xs, hc, w, 1e-5, cdt, S), tol)
    close(H.streams_norm(xs, None, w, 1e-5, cdt, S, row_idx=idx), R.streams_norm(xs, None, w, 1e-5, cdt, S, row_idx=idx), tol)
    y = torch.randn(T, D, device=DEV)
    z = torch.randn(T, D + 24, device=DEV)
    gate = z[:, 8:8 + D]
    for g in (gate, None):
        a, b = xs.clone(), xs.clone()
        close(H.streams_update_(a, y, g, hc, 0.45, S), R.streams_update_(b, y, g, hc, 0.45, S), 1e-5)
        a, b = xs.clone(), xs.clone()
        hc2 = torch.randn(2 * S + S * S, device=DEV)
        close(H.streams_update_norm_(a, y, g, hc, 0.45, S, hc2, w, 1e-5, cdt), R.streams_update_norm_(b, y, g, hc, 0.45, S, hc2, w, 1e-5, cdt), tol)
        close(a, b, 1e-5)
    if S == 1:
        a, b = xs.clone(), xs.clone()
        close(H.streams_update_norm_(a, y, gate, None, 0.7, 1, None, w, 1e-5, cdt), R.streams_update_norm_(b, y, gate, None, 0.7, 1, None, w, 1e-5, cdt), tol)
        close(a, b, 1e-5)
    table, ptab = torch.randn(50, D, device=DEV).to(cdt), torch.randn(90, D, device=DEV).to(cdt)
    ids = torch.randint(0, 50, (T,), dtype=torch.int32, device=DEV)
    pos = torch.randint(0, 90, (T,), dtype=torch.int32, device=DEV)
    close(H.embed_rows(ids, table, pos_table=ptab, tok_pos=pos, copies=S), R.embed_rows(ids, table, pos_table=ptab, tok_pos=pos, copies=S), 1e-6)
    close(H.embed_rows(ids, table, scale=1.5, copies=S), R.embed_rows(ids, table, scale=1.5, copies=S), 1e-6)
    lg = torch.randn(T, 70, device=DEV)
    close(H.scale_(lg.clone(), 0.25), R.scale_(lg.clone(), 0.25), 1e-7)
    o = torch.randn(T, D, device=DEV)
    close(H.sigmoid_gate(o, y, cdt), R.sigmoid_gate(o, y, cdt), tol)
    close(H.sigmoid_gate(o.to(cdt), y, cdt), R.sigmoid_gate(o.to(cdt), y, cdt), tol)
    close(H.unary(o, "gelu", cdt), R.unary(o, "gelu", cdt), tol)


@pytest.mark.parametrize("cdt,tol", DTYPES)
def test_rotation_in_halves_with_turn_count_rescaling(ops, cdt, tol):
    """Pairs (i, i + dims / 2) with frequencies rescaled by turn counts and amplified cosines and sines, with and
    without the norm in front, over part of a head and over heads wider than a wave, into a pool and in place."""
    H, R = ops
    torch.manual_seed(4)
    md, n_pages, _ = meta_of([40, 3, 1], [0, 77, 1200], DEV)
    T = 44
    sc = ("turns", 3.0, 300.0, 20.0, 2.0)
    for heads, n, dims in ((3, 32, 32), (2, 24, 10), (1, 200, 160), (4, 8, 8)):
        x = torch.randn(T, heads * n + 6, device=DEV)
        w = 1 + 0.2 * torch.randn(n, device=DEV)
        for ww in (w, None):
            a, b = torch.zeros(T, heads * n, device=DEV, dtype=cdt), torch.zeros(T, heads * n, device=DEV, dtype=cdt)
            kw = dict(w=ww, eps=1e-5, rot=(dims, 1e4, sc), half=True)
            close(H.head_norm_rope(x, heads, n, 3, n, a, 0, n, md, **kw), R.head_norm_rope(x, heads, n, 3, n, b, 0, n, md, **kw), tol)
        pa = torch.zeros(n_pages * 16, n + 5, device=DEV, dtype=cdt)
        pb = pa.clone()
        kw = dict(rot=(dims, 1e4, sc), half=True, row_map=md["kv_slot"])
        close(H.head_norm_rope(x, 1, n, 0, 0, pa, 5, 0, md, **kw), R.head_norm_rope(x, 1, n, 0, 0, pb, 5, 0, md, **kw), tol)
        xa, xb = x.clone(), x.clone()                                   # in place: every pair is read before it is written
        kw = dict(rot=(dims, 50.0), half=True)
        close(H.head_norm_rope(xa, heads, dims, n - dims, n, xa, n - dims, n, md, **kw), R.head_norm_rope(xb, heads, dims, n - dims, n, xb, n - dims, n, md, **kw), 1e-5)
    f = R.rope_freqs(32, 1e6, "cpu", sc)
    f0 = R.rope_freqs(32, 1e6, "cpu")
    assert f[0] == f0[0] and abs(float(f[-1] / f0[-1]) - 1 / 3) < 1e-6 and abs(R.rope_amp(sc) - (0.1 * np.log(3.0) + 1)) < 1e-12


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("Hh,G,d,dv", [(6, 2, 10, 14), (2, 2, 32, 48), (4, 2, 64, 128), (2, 1, 128, 64)])
def test_two_score_maps_over_shared_values_and_their_combine(ops, cdt, tol, Hh, G, d, dv):
    """Differential attention's pieces: 2 H query heads over 2 G key heads whose value head is the key head
    modulo G, fp32 outputs over pools of the GEMM type (prompt rows over tiles and decoded rows over long
    contexts with split keys), then the combine a1 - lambda a2 with its unit norm."""
    H, R = ops
    torch.manual_seed(Hh * d)
    for lens, pos0 in (([150, 17], [0, 0]), ([1, 1], [700, 45]), ([5, 40], [3, 90])):
        md, n_pages, _ = meta_of(lens, pos0, DEV)
        T = sum(lens)
        kc = (torch.randn(n_pages, 16, 2 * G * d, device=DEV) * 0.5).to(cdt)
        vc = torch.randn(n_pages, 16, G * dv, device=DEV).to(cdt)
        q = torch.randn(T, 2 * Hh * d, device=DEV)
        kw = dict(scale=d ** -0.5, softcap=0.0, r1=None, r2=None, chunk=0, page_size=16, out_dtype=cdt, v_heads=G)
        a, b = torch.empty(T, 2 * Hh * dv, device=DEV), torch.empty(T, 2 * Hh * dv, device=DEV)
        H.attn_paged(q, kc, vc, md, 2 * Hh, 2 * G, d, dv, out=a, **kw)
        R.attn_paged(q, kc, vc, md, 2 * Hh, 2 * G, d, dv, out=b, **kw)
        close(a, b, 2e-5 if cdt == torch.float32 else 1e-2)
        lam = 0.4 * torch.randn(4, d, device=DEV)
        close(H.diff_combine(b, lam, 0.35, Hh, dv, 1e-6, cdt), R.diff_combine(b, lam, 0.35, Hh, dv, 1e-6, cdt), tol)


@pytest.mark.parametrize("heads,dim,vdim", [(3, 7, 9), (5, 48, 72), (1, 1, 1), (2, 130, 70), (4, 128, 128), (1, 256, 300)])
def test_hgrn2_scan_carries_state(ops, heads, dim, vdim):
    """The gated recurrence over a batch of unequal requests, some continuing from carried states in scattered
    slots (prompt portions and single decoded rows), with and without the gate's bias; outputs and states."""
    H, R = ops
    torch.manual_seed(heads + dim)
    for lens, pos0 in (([33, 1, 7], [0, 5, 12]), ([1, 1, 1], [4, 0, 9]), ([70], [0])):
        md, _, n_slots = meta_of(lens, pos0, DEV)
        T = sum(lens)
        z = torch.randn(T, 2 * heads * dim + heads * vdim + 5, device=DEV)
        q, f, v = z[:, :heads * dim], z[:, heads * dim:2 * heads * dim], z[:, 2 * heads * dim:2 * heads * dim + heads * vdim]
        fb = torch.randn(heads * dim, device=DEV)
        lower = torch.rand(heads * dim, device=DEV)
        nw = 1 + 0.2 * torch.randn(vdim, device=DEV)
        st = torch.randn(n_slots, heads, dim, vdim, device=DEV)
        for bias in (fb, None):
            s1, s2 = st.clone(), st.clone()
            a = H.hgrn2_scan(q, f, v, bias, lower, nw, s1, md, heads, dim, vdim, 1e-5, torch.float32)
            b = R.hgrn2_scan(q, f, v, bias, lower, nw, s2, md, heads, dim, vdim, 1e-5, torch.float32)
            close(a, b, 2e-4)
            close(s1[md["slot"].long()], s2[md["slot"].long()], 2e-4)


@pytest.mark.parametrize("T,E,top,groups,keep", [(50, 8, 2, 4, 3), (7, 12, 3, 4, 2), (300, 5, 2, 5, 3), (33, 6, 6, 2, 2), (20, 7, 1, 0, 0),
                                                 (64, 64, 8, 8, 4), (9, 128, 16, 64, 9)])
def test_grouped_sigmoid_routing(ops, T, E, top, groups, keep):
    H, R = ops
    torch.manual_seed(T + E)
    logits = torch.randn(T, E + 3, device=DEV)[:, 1:1 + E] * 2
    a, b = H.moe_route_grouped(logits, top, groups, keep, 1.9), R.moe_route_grouped(logits, top, groups, keep, 1.9)
    assert torch.equal(a.ids.cpu().sort(-1).values, b.ids.cpu().sort(-1).values)
    assert torch.equal(a.ids.cpu(), b.ids.cpu())
    close(a.w, b.w, 1e-5)
    assert torch.equal(a.offs.cpu(), b.offs.cpu())
    assert torch.equal(a.rows.cpu().long().bincount(minlength=T), torch.full((T,), top))
    # every (token, choice) sits in its expert's range of sorted rows
    offs, dest = a.offs.cpu().long(), a.dest.cpu().long()
    assert bool(((dest >= offs[a.ids.cpu().long()]) & (dest < offs[a.ids.cpu().long() + 1])).all())
    assert torch.equal(a.rows.cpu().long()[dest], torch.arange(T)[:, None].expand(T, top))


@pytest.mark.parametrize("cdt,tol", DTYPES)
@pytest.mark.parametrize("Hh,G,Gv,d,dv,rot", [(12, 4, 2, 10, 14, (6, 50.0)), (8, 4, 2, 64, 128, (32, 1e6)), (2, 2, 1, 32, 64, (32, 1e4)),
                                              (4, 2, 1, 130, 70, None)])
def test_projected_rows_with_weighted_norms_before_the_rotation(ops, cdt, tol, Hh, G, Gv, d, dv, rot):
    """The one-pass kernel in its second form: q and k heads RMS-normed with a weight before the rotation, fewer
    value heads than key heads in the row, no convolution; against the chain of plain ops."""
    H, R = ops
    torch.manual_seed(21)
    C = Hh * d + G * d + Gv * dv
    qw, kw_ = 1 + 0.3 * torch.randn(d, device=DEV), 1 + 0.3 * torch.randn(d, device=DEV)
    for lens, pos0 in (([1, 40, 3, 130], [900, 0, 17, 2000]), ([1, 1, 1], [5, 0, 300])):
        md, n_pages, _ = meta_of(lens, pos0, DEV)
        T = sum(lens)
        z = torch.randn(T, C + 7, device=DEV)
        outs = []
        for O in (H, R):
            q = torch.zeros(T, Hh * d, device=DEV)
            kc = torch.zeros(n_pages, 16, G * d, device=DEV, dtype=cdt)
            vc = torch.zeros(n_pages, 16, Gv * dv, device=DEV, dtype=cdt)
            O.qkv_conv_rope_store(z, None, None, md, Hh, G, d, dv, q, kc, vc, eps=1e-5, rot=rot, v_heads=Gv, q_norm=qw, k_norm=kw_)
            outs.append((q, kc, vc))
        close(outs[0][0], outs[1][0], 3e-4)
        close(outs[0][1], outs[1][1], max(tol, 3e-4))
        close(outs[0][2], outs[1][2], tol)
