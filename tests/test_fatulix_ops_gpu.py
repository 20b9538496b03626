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
    H.moe_route(h, wr, idx, wt, T, W, E, top, f32)
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


def _diffattn_ref(q, k, v, gate, scale, lam, out_scale, eps):
    """q [T][H][2][D], k [T][G][2][D], v [T][G][Dv] (one sequence, causal), float64."""
    T, Hh, _, D = q.shape
    G = k.shape[1]
    mask = torch.ones(T, T, dtype=torch.bool, device=q.device).tril()
    out = []
    for h in range(Hh):
        kv = h // (Hh // G)
        a = [torch.softmax(((q[:, h, m] @ k[:, kv, m].T) * scale).masked_fill(~mask, float("-inf")), -1) @ v[:, kv] for m in range(2)]
        o = a[0] - lam * a[1]
        o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + eps) * out_scale * gate[:, h:h + 1]
        out.append(o)
    return torch.cat(out, -1)


@pytest.mark.parametrize("f32", MODES)
@pytest.mark.parametrize("Hh,G,D,Dv,bs", [(4, 2, 56, 80, 64), (3, 3, 20, 24, 16), (6, 1, 64, 40, 32), (2, 2, 136, 520 - 8, 64)])
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
    kc = torch.zeros(nblk, G, bs, 2 * D, dtype=el, device=DEV)
    vc = torch.zeros(nblk, G, bs, Dv, dtype=el, device=DEV)
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
    torch.testing.assert_close(vc[blk, :, off].double(), v_ref, **_tol(f32))
    out = torch.zeros(T, Hh * Dv, dtype=el, device=DEV)
    cu = torch.tensor([0, T], dtype=torch.int32, device=DEV)
    H.diffattn_paged(qo, kc, vc, gate, bt, nblk, pos, 1, T, Hh, G, D, Dv, bs, scale, lam, osc, eps, out, f32, cu_q=cu)
    # the reference attends over what the cache holds (the stored roundings), so only the attention arithmetic is compared
    ref = _diffattn_ref(qo.double().view(T, Hh, 2, D), kc[blk, :, off].double().view(T, G, 2, D), vc[blk, :, off].double(), gate.double(),
                        scale, lam, osc, eps)
    torch.testing.assert_close(out.double(), ref, **(dict(rtol=1e-4, atol=1e-4) if f32 else dict(rtol=1.6e-2, atol=1.6e-2)))
