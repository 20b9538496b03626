"""Every kernel of the fp32-residual / differential-attention / routed feed-forward family through the C ABI, one mechanism at a
time, against plain PyTorch fp32 statements of the same operation -- in bf16 and in fp32 element mode, at sizes that are NOT multiples
of the tiles (odd widths, head sizes that are no power of two, K not a multiple of 8)."""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda"
MODES = [False, True]       # f32 element mode


def _elem(f32):
    return torch.float32 if f32 else torch.bfloat16


def _rand(shape, f32, gen, scale=1.0):
    """Values exactly representable in the element type (so the fp32 reference sees the kernel's inputs)."""
    return (torch.randn(*shape, generator=gen) * scale).to(_elem(f32)).to(DEV)


def _tol(f32):
    return dict(rtol=2e-5, atol=2e-5) if f32 else dict(rtol=1.6e-2, atol=1.6e-2)


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("M,N,K", [(1, 7, 5), (3, 64, 32), (23, 100, 72), (130, 193, 260), (64, 440, 264), (5, 33, 1000)])
@pytest.mark.parametrize("epi", [0, 1, 2])
def test_gemm_rows(f32, M, N, K, epi):
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(M * 1000 + N + K)
    x, w = _rand((M, K), f32, g), _rand((N, K), f32, g, 1 / math.sqrt(K))
    y = torch.full((M, N), float("nan"), dtype=torch.float32 if epi == 0 else _elem(f32), device=DEV)
    H.gemm_rows(x, w, y, M, N, K, f32, epi)
    ref = x.double() @ w.double().T
    if epi == 1:
        ref = torch.relu(ref) ** 2
    torch.testing.assert_close(y.double(), ref, **(_tol(f32) if epi else dict(rtol=2e-5, atol=2e-5)))


@pytest.mark.parametrize("f32", MODES)
def test_gemm_rows_grouped_gathers_rows_and_never_mixes_groups(f32):
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(5)
    T, top, E, N, K = 37, 3, 5, 50, 44
    x = _rand((T, K), f32, g)
    w = _rand((E, N, K), f32, g, 1 / math.sqrt(K))
    counts = [70, 0, 1, 30, 10]                     # one group larger than a tile, one empty, one single row
    assert sum(counts) == T * top
    off = torch.tensor([0] + list(torch.tensor(counts).cumsum(0)), dtype=torch.int32, device=DEV)
    perm = torch.randperm(T * top, generator=g).to(torch.int32).to(DEV)
    y = torch.full((T * top, N), float("nan"), dtype=torch.float32, device=DEV)
    H.gemm_rows_grouped(x, w, y, off, E, T * top, N, K, f32, 0, row_idx=perm, idx_div=top)
    r0 = 0
    for e, c in enumerate(counts):
        rows = (perm[r0:r0 + c] // top).long()
        torch.testing.assert_close(y[r0:r0 + c].double(), x[rows].double() @ w[e].double().T, rtol=2e-5, atol=2e-5)
        r0 += c


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("W", [64, 200, 1030])
def test_sandwich_norms_and_embedding(f32, W):
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(W)
    T, V, eps = 9, 31, 1e-5
    table = _rand((V, W), f32, g)
    ids = torch.randint(0, V, (T,), generator=g).to(DEV)
    x, x0 = torch.zeros(T, W, device=DEV), torch.zeros(T, W, device=DEV)
    H.embed_res32(ids, table, x, x0, T, W, f32)
    assert torch.equal(x, table[ids].float()) and torch.equal(x0, x)
    w = _rand((W,), f32, g) + 1
    x = torch.randn(T, W, generator=g).to(DEV) * 3
    add = torch.randn(T, W, generator=g).to(DEV)
    xin = x.clone()
    out = torch.zeros(T, W, dtype=_elem(f32), device=DEV)
    H.rmsnorm_res32(x, w, eps, out, T, W, f32, add=add)
    s = (xin + add).double()
    assert torch.equal(x, xin + add)
    ref = s / torch.sqrt((s * s).mean(-1, keepdim=True) + eps) * w.double()
    torch.testing.assert_close(out.double(), ref, **_tol(f32))
    gather = torch.tensor([4, 0, 8], dtype=torch.int32, device=DEV)
    out2 = torch.zeros(3, W, dtype=_elem(f32), device=DEV)
    H.rmsnorm_res32(x, w, eps, out2, 3, W, f32, gather=gather)
    torch.testing.assert_close(out2.double(), ref[gather.long()], **_tol(f32))
    y = torch.randn(T, W, generator=g).to(DEV) * 7
    x1 = x.clone()
    H.rmsnorm_add_res32(y, w, eps, x1, T, W, f32)
    yd = y.double()
    torch.testing.assert_close(x1.double(), x.double() + yd / torch.sqrt((yd * yd).mean(-1, keepdim=True) + eps) * w.double(), rtol=1e-5, atol=1e-5)


def test_rows_f32_to_bf16_pads_with_minus_infinity():
    from ssd_amd.hip import ops as H
    src = torch.randn(3, 13, device=DEV)
    dst = torch.zeros(3, 16, dtype=torch.bfloat16, device=DEV)
    H.rows_f32_to_bf16(src, dst, 3, 13, 13, 16)
    assert torch.equal(dst[:, :13], src.to(torch.bfloat16)) and torch.isinf(dst[:, 13:]).all() and (dst[:, 13:] < 0).all()


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("E,top", [(7, 2), (5, 1), (6, 6), (70, 4)])
def test_route_plan_combine(f32, E, top):
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(E * 10 + top)
    T, W = 29, 72
    h, wr = _rand((T, W), f32, g), _rand((E, W), f32, g, 1 / math.sqrt(W))
    idx = torch.zeros(T, top, dtype=torch.int32, device=DEV)
    wt = torch.zeros(T, top, device=DEV)
    zl = torch.zeros(T, E, device=DEV)
    H.gemm_rows(h, wr, zl, T, E, W, f32)
    H.moe_route(zl, idx, wt, T, E, top)
    z = h.double() @ wr.double().T
    val, ref_idx = z.topk(top, dim=-1)
    assert torch.equal(idx.long(), ref_idx)                      # random logits: no close calls
    torch.testing.assert_close(wt.double(), torch.softmax(val, -1), rtol=1e-5, atol=1e-6)
    off = torch.zeros(E + 1, dtype=torch.int32, device=DEV)
    perm = torch.zeros(T * top, dtype=torch.int32, device=DEV)
    inv = torch.zeros(T * top, dtype=torch.int32, device=DEV)
    H.moe_plan(idx, T, top, E, off, perm, inv)
    flat = idx.view(-1).long()
    assert off.tolist() == [0] + torch.bincount(flat, minlength=E).cumsum(0).tolist()
    assert sorted(perm.tolist()) == list(range(T * top)) and torch.equal(perm[inv.long()].long(), torch.arange(T * top, device=DEV))
    for e in range(E):
        assert (flat[perm[off[e]:off[e + 1]].long()] == e).all()
    y = torch.randn(T * top, W, generator=g).to(DEV)
    sh = torch.randn(T, W, generator=g).to(DEV)
    out = torch.zeros(T, W, device=DEV)
    H.moe_combine(y, inv, wt, sh, out, T, top, W)
    ref = (wt.double().unsqueeze(-1) * y[inv.long()].view(T, top, W).double()).sum(1) + sh.double()
    torch.testing.assert_close(out.double(), ref, rtol=1e-5, atol=1e-5)


def _paged_ref(qo, kc, vt, gate, bt, pos, seq, Hh, G, D, Dv, bs, scale, lam, osc, eps):
    """Token by token from what the CACHE holds (K [blk][G][bs][2D], V^T [blk][G][Dv][bs]): float64, keys 0 .. pos[t] of sequence seq[t]."""
    T = qo.shape[0]
    q = qo.double().view(T, Hh, 2, D)
    out = torch.zeros(T, Hh * Dv, dtype=torch.float64, device=qo.device)
    for t in range(T):
        n = int(pos[t]) + 1
        j = torch.arange(n, device=qo.device)
        pg = bt[int(seq[t])].long()[j // bs]
        K = kc[pg, :, j % bs].double().view(n, G, 2, D)
        V = vt[pg, :, :, j % bs].double()                       # [n][G][Dv]
        for h in range(Hh):
            g = h // (Hh // G)
            a = [torch.softmax((K[:, g, m] @ q[t, h, m]) * scale, 0) @ V[:, g] for m in range(2)]
            o = a[0] - lam * a[1]
            out[t, h * Dv:(h + 1) * Dv] = o / torch.sqrt((o * o).mean() + eps) * osc * gate[t, h].double()
    return out


SHAPES = [(4, 2, 56, 80, 64), (8, 2, 64, 128, 32), (4, 4, 128, 64, 64), (5, 5, 8, 16, 32), (6, 2, 16, 32, 32),   # the MFMA form takes these in bf16
          (3, 3, 20, 24, 16), (6, 1, 64, 40, 32), (2, 2, 136, 512 - 8, 64)]                          # scalar form only


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("Hh,G,D,Dv,bs", SHAPES)
def test_diffattn_store_and_paged_over_scattered_pages(f32, Hh, G, D, Dv, bs):
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(D + Dv)
    T, eps, scale, lam, osc = 150, 1e-5, 0.21, 0.37, 0.7
    el = _elem(f32)
    N = Hh * 2 * D + G * 2 * D + G * Dv + Hh
    qkvg = (torch.randn(T, N, generator=g) * 1.5).to(DEV)
    qw, kw = _rand((D,), f32, g) + 1, _rand((D,), f32, g) + 1
    nblk = 16
    pages = torch.randperm(nblk, generator=g)[: -(-T // bs)].tolist()
    bt = torch.full((1, nblk), -1, dtype=torch.int32)
    bt[0, :len(pages)] = torch.tensor(pages, dtype=torch.int32)
    bt = bt.to(DEV)
    pos = torch.arange(T, dtype=torch.int64, device=DEV)
    slots = torch.tensor([pages[p // bs] * bs + p % bs for p in range(T)], dtype=torch.int32, device=DEV)
    kc = torch.full((nblk, G, bs, 2 * D), float("nan"), dtype=el, device=DEV)
    vc = torch.full((nblk, G, Dv, bs), float("nan"), dtype=el, device=DEV)
    qo = torch.zeros(T, Hh * 2 * D, dtype=el, device=DEV)
    gate = torch.zeros(T, Hh, device=DEV)
    H.diffattn_store(qkvg, qw, kw, eps, slots, qo, gate, kc, vc, T, Hh, G, D, Dv, bs, f32)
    x = qkvg.double()
    nq, nk, nv = Hh * 2 * D, G * 2 * D, G * Dv
    rms = lambda t: t / torch.sqrt((t * t).mean(-1, keepdim=True) + eps)
    q_ref = rms(x[:, :nq].view(T, Hh, 2, D)) * qw.double()
    k_ref = rms(x[:, nq:nq + nk].view(T, G, 2, D)) * kw.double()
    v_ref = x[:, nq + nk:nq + nk + nv].view(T, G, Dv)
    torch.testing.assert_close(qo.double().view(T, Hh, 2, D), q_ref, **_tol(f32))
    torch.testing.assert_close(gate.double(), torch.sigmoid(x[:, nq + nk + nv:]), rtol=1e-5, atol=1e-6)
    blk, off = (slots // bs).long(), (slots % bs).long()
    torch.testing.assert_close(kc[blk, :, off].double().view(T, G, 2, D), k_ref, **_tol(f32))
    torch.testing.assert_close(vc[blk, :, :, off].double(), v_ref, **_tol(f32))
    # keys that stand out, far back and at page borders: map 1 of head 0 looks at key 0 from every later position, map 2 at the last
    # key of the first page; a key that is skipped or mixed up is an O(1) error
    qn = qo.double().view(T, Hh, 2, D)
    kc[pages[0], 0, 0, :D] = (6 * qn[T - 1, 0, 0] / qn[T - 1, 0, 0].norm() * D ** 0.5).to(el)
    kc[pages[0], 0, bs - 1, D:] = (6 * qn[T - 1, 0, 1] / qn[T - 1, 0, 1].norm() * D ** 0.5).to(el)
    seq = torch.zeros(T, dtype=torch.int64)
    ref = _paged_ref(qo, kc, vc, gate, bt, pos, seq, Hh, G, D, Dv, bs, scale, lam, osc, eps)
    tol = dict(rtol=1e-4, atol=1e-4) if f32 else dict(rtol=2e-2, atol=2e-2)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    ctx = torch.tensor([T], dtype=torch.int32, device=DEV)
    for fast in (False, True):          # the scalar form, then (where the shape allows it in bf16) the MFMA form
        out = torch.zeros(T, Hh * Dv, dtype=el, device=DEV)
        H.diffattn_paged(qo, kc, vc, gate, bt, nblk, pos, 1, T, Hh, G, D, Dv, bs, scale, lam, osc, eps, out, f32, cu_q=cu,
                         **(dict(context_lens=ctx, max_q=T) if fast else {}))
        torch.testing.assert_close(out.double(), ref, **tol)


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("Hh,G,D,Dv,bs", SHAPES[:6])
def test_diffattn_decode_rows_of_several_sequences(f32, Hh, G, D, Dv, bs):
    """A batch of sequences with different lengths bringing one or two rows each (decoding, the last tokens of a portion): keys just
    inside the visible range count, the key after a row's position does not (the second row's key is in the cache when the first row
    attends), page borders fall at and next to the positions, unwritten slots hold NaN."""
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(Hh * 100 + D)
    eps, scale, lam, osc = 1e-6, 0.3, 0.45, 0.9
    el = _elem(f32)
    lens = [bs + 1, 2 * bs, 1, 3 * bs - 1, 2]             # context lengths INCLUDING the new rows
    new = [1, 2, 1, 2, 2]
    B, nblk = len(lens), 16
    order = torch.randperm(nblk, generator=g).tolist()
    bt = torch.full((B, nblk), -1, dtype=torch.int32)
    tables, at = [], 0
    for b, n in enumerate(lens):
        k = -(-n // bs)
        tables.append(order[at:at + k]); at += k
        bt[b, :k] = torch.tensor(tables[-1], dtype=torch.int32)
    bt = bt.to(DEV)
    kc = torch.full((nblk, G, bs, 2 * D), float("nan"), dtype=el, device=DEV)
    vc = torch.full((nblk, G, Dv, bs), float("nan"), dtype=el, device=DEV)
    N = Hh * 2 * D + G * 2 * D + G * Dv + Hh
    qw, kw = _rand((D,), f32, g) + 1, _rand((D,), f32, g) + 1
    # fill every sequence's context through the store kernel, then the rows of this step are its last `new` tokens
    rows_q, rows_gate, pos, seq = [], [], [], []
    for b, n in enumerate(lens):
        x = (torch.randn(n, N, generator=g) * 1.5).to(DEV)
        slots = torch.tensor([tables[b][p // bs] * bs + p % bs for p in range(n)], dtype=torch.int32, device=DEV)
        qo = torch.zeros(n, Hh * 2 * D, dtype=el, device=DEV)
        gt = torch.zeros(n, Hh, device=DEV)
        H.diffattn_store(x, qw, kw, eps, slots, qo, gt, kc, vc, n, Hh, G, D, Dv, bs, f32)
        rows_q.append(qo[n - new[b]:]); rows_gate.append(gt[n - new[b]:])
        pos += list(range(n - new[b], n)); seq += [b] * new[b]
    q, gate = torch.cat(rows_q).contiguous(), torch.cat(rows_gate).contiguous()
    T = q.shape[0]
    posd = torch.tensor(pos, dtype=torch.int64, device=DEV)
    cu = torch.tensor([0] + torch.tensor(new).cumsum(0).tolist(), dtype=torch.int32, device=DEV)
    ctx = torch.tensor(lens, dtype=torch.int32, device=DEV)
    ref = _paged_ref(q, kc, vc, gate, bt, posd, torch.tensor(seq), Hh, G, D, Dv, bs, scale, lam, osc, eps)
    tol = dict(rtol=1e-4, atol=1e-4) if f32 else dict(rtol=2e-2, atol=2e-2)
    ws = torch.zeros(256 * 4160, device=DEV)
    for kw in ({}, dict(context_lens=ctx, max_q=2), dict(context_lens=ctx, max_q=2, workspace=ws, ctx_hint=4096)):
        # the scalar form; the MFMA form (where the shape allows it in bf16); the same with the keys cut into slices over the grid
        # (more slices than some sequences have steps: empty slices must merge as nothing)
        out = torch.zeros(T, Hh * Dv, dtype=el, device=DEV)
        H.diffattn_paged(q, kc, vc, gate, bt, nblk, posd, B, T, Hh, G, D, Dv, bs, scale, lam, osc, eps, out, f32, cu_q=cu, **kw)
        torch.testing.assert_close(out.double(), ref, **tol)


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("routed", [False, True])
@pytest.mark.parametrize("W", [200, 2048])          # 2048: few rows of a wide model take the 1024-thread form (another summation order)
def test_sandwich_tail_equals_its_separate_launches(f32, routed, W):
    from ssd_amd.hip import ops as H
    g = torch.Generator().manual_seed(11)
    T, top, eps = 7, 3, 1e-5
    el = _elem(f32)
    wp, wn = _rand((W,), f32, g) + 1, _rand((W,), f32, g) + 1
    x0 = torch.randn(T, W, generator=g).to(DEV)
    add = torch.randn(T, W, generator=g).to(DEV)
    ydn = torch.randn(T * top, W, generator=g).to(DEV)
    sh = torch.randn(T, W, generator=g).to(DEV)
    inv = torch.randperm(T * top, generator=g).to(torch.int32).to(DEV)
    wt = torch.rand(T, top, generator=g).to(DEV)
    y = torch.randn(T, W, generator=g).to(DEV)
    # separate launches
    xa = x0.clone()
    if routed:
        y = torch.zeros(T, W, device=DEV)
        H.moe_combine(ydn, inv, wt, sh, y, T, top, W)
    H.rmsnorm_add_res32(y, wp, eps, xa, T, W, f32)
    na = torch.zeros(T, W, dtype=el, device=DEV)
    H.rmsnorm_res32(xa, wn, eps, na, T, W, f32, add=add)
    # one launch
    xb, nb, scratch = x0.clone(), torch.zeros(T, W, dtype=el, device=DEV), torch.zeros(T, W, device=DEV)
    src = dict(ydn=ydn, inv=inv, weights=wt, shared=sh, top=top, y_scratch=scratch) if routed else dict(y=y)
    H.sandwich_tail(wp, eps, xb, T, W, f32, next_add=add, next_weight=wn, next_out=nb, **src)
    torch.testing.assert_close(xb, xa, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(nb.float(), na.float(), **(dict(rtol=1e-5, atol=1e-5) if f32 else dict(rtol=1e-2, atol=1e-2)))
    xc = x0.clone()                     # the last sublayer of a model: no next norm
    H.sandwich_tail(wp, eps, xc, T, W, f32, **src)
    xd = x0.clone()
    H.rmsnorm_add_res32(y, wp, eps, xd, T, W, f32)
    torch.testing.assert_close(xc, xd, rtol=1e-5, atol=1e-5)
