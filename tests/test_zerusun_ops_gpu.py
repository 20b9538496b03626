"""The HIP kernels behind the Zerusun decoder, one mechanism at a time, against plain fp32 / fp64 torch statements of the same op:
Dynamic-Tanh rows and the parallel layer's tail, GLU rows, the batched per-head GEMM, the softmax router with group-limited choice,
the latent cache store + windowed attention over scattered pages, the linear-attention scan over state slots in portions."""
import math

import pytest
import torch

from oracle import zerusun as Z

pytestmark = pytest.mark.gpu
DEV = "cuda"


def H():
    from ssd_amd.hip import ops
    return ops


def rnd(*shape, seed=0, scale=1.0):
    return (torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale)


def elem(f32):
    return torch.float32 if f32 else torch.bfloat16


def tol(f32):
    return dict(rtol=2e-5, atol=2e-5) if f32 else dict(rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("W", [40, 328])
def test_dyt_embed_rows_and_parallel_tail(f32, W):
    T, V, top = 9, 23, 3
    el = elem(f32)
    table, w, b = (rnd(V, W, seed=1).to(el), (1 + 0.1 * rnd(W, seed=2)).to(el), (0.1 * rnd(W, seed=3)).to(el))
    alpha = torch.tensor([0.7])
    ids = torch.randint(0, V, (T,), generator=torch.Generator().manual_seed(4))
    x, x0 = torch.zeros(T, W, device=DEV), torch.zeros(T, W, device=DEV)
    cat = torch.zeros(T * 2 * W, dtype=el, device=DEV)
    d = lambda t: t.to(DEV)
    H().dyt_embed(d(ids), d(table), d(alpha), d(w), d(b), x, x0, cat[W:], 2 * W, T, W, f32)
    ref = Z.dyt(table.double()[ids], w.double(), b.double(), 0.7)
    assert torch.allclose(x.cpu().double(), ref, **tol(True)) and torch.equal(x, x0)
    assert torch.allclose(cat.view(T, 2 * W)[:, W:].cpu().double(), ref, **tol(f32)) and float(cat.view(T, 2 * W)[:, :W].abs().max()) == 0
    # rows with a vector added first, and a gather
    add = (0.3 * rnd(W, seed=5)).to(el)
    out = torch.zeros(T, W, dtype=el, device=DEV)
    x1 = x.clone()
    H().dyt_rows(x1, d(alpha), d(w), d(b), out, T, W, f32, add_vec=d(add))
    assert torch.allclose(x1.cpu().double(), ref + add.double(), **tol(True))
    assert torch.allclose(out.cpu().double(), Z.dyt(ref + add.double(), w.double(), b.double(), 0.7), **tol(f32))
    g = torch.tensor([5, 0, 8], dtype=torch.int32)
    out3 = torch.zeros(3, W, dtype=el, device=DEV)
    H().dyt_rows(x, d(alpha), d(w), d(b), out3, 3, W, f32, gather=d(g))
    assert torch.allclose(out3.cpu().double(), Z.dyt(ref[g.long()], w.double(), b.double(), 0.7), **tol(f32))
    # the tail: x += mix + (dense | routed + gated shared | nothing), then the next norm or the [x | x0] copy
    y_mix, y_ff, ydn, ysh = rnd(T, W, seed=6), rnd(T, W, seed=7), rnd(T * top, W, seed=8), rnd(T, W, seed=9)
    wt, sg = rnd(T, top, seed=10).abs(), rnd(T, 5, seed=11)
    inv = torch.randperm(T * top, generator=torch.Generator().manual_seed(12)).to(torch.int32)
    routed = (wt.double()[..., None] * ydn.double()[inv.long()].view(T, top, W)).sum(1) + torch.sigmoid(sg.double()[:, 4:5]) * ysh.double()
    for ff, kw in ((y_ff.double(), dict(y_ff=d(y_ff))), (torch.zeros(T, W).double(), {}),
                   (routed, dict(ydn=d(ydn), inv=d(inv), weights=d(wt), top=top, shared=d(ysh), shared_gate=d(sg).view(-1)[4:], ld_shared_gate=5))):
        xa, nxt, cat2 = x.clone(), torch.zeros(T, W, dtype=el, device=DEV), torch.zeros(T * 2 * W, dtype=el, device=DEV)
        H().parallel_tail(xa, d(y_mix), T, W, f32, next_alpha=d(alpha), next_weight=d(w), next_bias=d(b), next_out=nxt, cat=cat2,
                          ld_cat=2 * W, **kw)
        want = x.cpu().double() + (y_mix.double() + ff)
        assert torch.allclose(xa.cpu().double(), want, **tol(True))
        assert torch.allclose(nxt.cpu().double(), Z.dyt(want, w.double(), b.double(), 0.7), **tol(f32))
        assert torch.allclose(cat2.view(T, 2 * W)[:, :W].cpu().double(), want, **tol(f32))


@pytest.mark.parametrize("f32", [True, False])
def test_glu_rows_and_batched_gemm(f32):
    el = elem(f32)
    rows, F = 7, 52
    ab = rnd(rows, 2 * F, seed=1, scale=2.0)
    for act, fn in ((0, Z.silu), (1, Z.gelu_tanh)):
        out = torch.zeros(rows, F, dtype=el, device=DEV)
        H().glu_rows(ab.to(DEV), out, rows, F, act, f32)
        assert torch.allclose(out.cpu().double(), fn(ab[:, :F].double()) * ab[:, F:].double(), **tol(f32))
    # per-head products over column slices of token-major rows; few rows (the weight-streaming form in bf16) and many
    for M in (3, 150):
        G, K, N, extra = 5, 24, 40, 8
        x = rnd(M, G * (K + extra), seed=2).to(el)
        w = rnd(G, N, K, seed=3).to(el)
        y = torch.full((M, G * N + 3), 7.0, device=DEV)
        H().gemm_rows_batched(x.to(DEV), w.to(DEV), y, M, N, K, G, G * (K + extra), K + extra, G * N + 3, N, f32)
        ref = torch.einsum("mgk,gnk->mgn", x.double().view(M, G, K + extra)[..., :K], w.double()).reshape(M, G * N)
        assert torch.allclose(y[:, :G * N].cpu().double(), ref, **tol(f32)) and bool((y[:, G * N:] == 7.0).all())


@pytest.mark.parametrize("M", [1, 9, 200])
def test_gemm_with_the_glu_as_epilogue(M):
    """bf16: weight rows in (gate, up) pairs, output act(gate) * up -- the tile form, the skinny form, dense and per expert."""
    K, F, E = 72, 44, 3
    x = rnd(M, K, seed=1).bfloat16()
    gate, up = rnd(E, F, K, seed=2, scale=0.3).bfloat16(), rnd(E, F, K, seed=3, scale=0.3).bfloat16()
    pairs = torch.stack([gate, up], dim=2).reshape(E, 2 * F, K).contiguous()
    for epi, fn in ((H().GR_GLU_SILU, Z.silu), (H().GR_GLU_GELU, Z.gelu_tanh)):
        y = torch.zeros(M, F, dtype=torch.bfloat16, device=DEV)
        H().gemm_rows(x.to(DEV), pairs[0].contiguous().to(DEV), y, M, 2 * F, K, False, epi)
        ref = fn(x.double() @ gate[0].double().T) * (x.double() @ up[0].double().T)
        assert torch.allclose(y.cpu().double(), ref, rtol=2e-2, atol=2e-2)
    # grouped: rows sorted by expert
    cnt = [M // 3, 0, M - M // 3]
    off = torch.tensor([0, cnt[0], cnt[0], M], dtype=torch.int32)
    y = torch.zeros(M, F, dtype=torch.bfloat16, device=DEV)
    H().gemm_rows_grouped(x.to(DEV), pairs.to(DEV), y, off.to(DEV), E, M, 2 * F, K, False, H().GR_GLU_SILU)
    which = torch.tensor([0] * cnt[0] + [2] * cnt[2])
    ref = torch.stack([Z.silu(x[r].double() @ gate[which[r]].double().T) * (x[r].double() @ up[which[r]].double().T) for r in range(M)])
    assert torch.allclose(y.cpu().double(), ref, rtol=2e-2, atol=2e-2)
    with pytest.raises(Exception):
        H().gemm_rows(x.float().to(DEV), pairs[0].float().contiguous().to(DEV), y, M, 2 * F, K, True, H().GR_GLU_SILU)


@pytest.mark.parametrize("E,top,groups,keep", [(16, 4, 2, 1), (12, 3, 3, 2), (8, 2, 1, 1), (6, 6, 3, 3), (5, 1, 5, 1), (130, 8, 10, 3)])
def test_softmax_router_with_group_limited_choice(E, top, groups, keep):
    T, ld = 33, E + 1
    z = rnd(T, ld, seed=E, scale=2.0)
    idx = torch.zeros(T, top, dtype=torch.int32, device=DEV)
    wt = torch.zeros(T, top, device=DEV)
    H().moe_route_softmax(z.to(DEV), ld, idx, wt, T, E, top, groups, keep, 1.5)
    ri, rw = Z.route(z[:, :E].double(), {"top": top, "scale": 1.5, "groups": {"count": groups, "keep": keep}})
    assert torch.equal(idx.cpu().long(), ri)
    assert torch.allclose(wt.cpu().double(), rw, rtol=1e-5, atol=1e-7)


def _pages(n_seq, lens, bs, seed):
    """Scattered pages: block tables [n_seq][max_blocks] over a shuffled pool."""
    need = [-(-n // bs) for n in lens]
    pool = torch.randperm(sum(need) + 3, generator=torch.Generator().manual_seed(seed)).tolist()
    mb = max(need)
    bt, at = [], 0
    for n in need:
        bt.append(pool[at:at + n] + [-1] * (mb - n))
        at += n
    return torch.tensor(bt, dtype=torch.int32), mb, sum(need) + 3


@pytest.mark.parametrize("f32", [True, False])
@pytest.mark.parametrize("Hh,D,R,Cr,Qr,win,rd,bs", [(6, 32, 32, 128, 64, 40, 32, 64), (3, 8, 6, 20, 12, 5, 4, 16), (5, 16, 8, 72, 40, 0, 8, 16),
                                                    (1, 8, 2, 8, 8, 1, 2, 16), (20, 16, 64, 512, 32, 33, 48, 16), (17, 8, 32, 32, 16, 0, 32, 32),
                                                    (16, 8, 32, 288, 16, 32, 2, 16)])
@pytest.mark.parametrize("lens", [[37, 50], [333, 207]])
def test_latent_store_and_windowed_attention_over_scattered_pages(f32, Hh, D, R, Cr, Qr, win, rd, bs, lens):
    """Two sequences; the second arrives in two launches (a portion, then the rest) and must see the keys of the first launch.  Where the
    MFMA form takes the sizes (bf16, latent sizes in multiples of 32) it is the one that runs, with the latent-space queries as bf16 rows."""
    el = elem(f32)
    if lens[0] > 100:
        win = win * 5          # windows of many key steps, ending inside and at the borders of pages
    eps, scale = 1e-5, 0.2
    freqs, mag = Z.rope_frequencies(rd, 10000.0, {"factor": 4.0, "original": 32, "fast": 16.0, "slow": 1.0})
    NP = Qr + Cr + R + Hh
    bt, mb, nblk = _pages(2, lens, bs, 3)
    cache = torch.full((nblk * bs, Cr + R), float("nan"), dtype=el, device=DEV)
    wq, wkv = (1 + 0.1 * rnd(Qr, seed=1)).to(el), (1 + 0.1 * rnd(Cr, seed=2)).to(el)
    d = lambda t: t.to(DEV)
    fq = freqs.float()
    proj_all = [rnd(n, NP, seed=10 + i) for i, n in enumerate(lens)]
    q_all = [rnd(n, Hh * (D + R), seed=20 + i).to(el) for i, n in enumerate(lens)]
    qabs_all = [rnd(n, Hh * Cr, seed=30 + i) for i, n in enumerate(lens)]
    mfma = H().latent_attn_mfma_ok(Cr, R, f32)
    assert mfma == ((not f32) and Cr % 32 == 0 and R % 32 == 0)
    if mfma:
        qabs_all = [q.bfloat16() for q in qabs_all]
    # with a workspace and few rows the MFMA form cuts the window over several workgroups and merges the slices
    ws = torch.full((256 * (Cr * 16 + 32),), float("nan"), device=DEV) if mfma else None

    def launch(parts):
        """parts: [(seq, lo, hi)] -> out rows of all parts."""
        proj = torch.cat([proj_all[s][lo:hi] for s, lo, hi in parts])
        q = torch.cat([q_all[s][lo:hi] for s, lo, hi in parts])
        qa = torch.cat([qabs_all[s][lo:hi] for s, lo, hi in parts])
        pos = torch.cat([torch.arange(lo, hi) for s, lo, hi in parts])
        slots = torch.cat([torch.tensor([int(bt[s][p // bs]) * bs + p % bs for p in range(lo, hi)], dtype=torch.int32) for s, lo, hi in parts])
        cu = torch.tensor([0] + list(torch.tensor([hi - lo for _, lo, hi in parts]).cumsum(0)), dtype=torch.int32)
        T = proj.shape[0]
        cq, gate = torch.zeros(T, Qr, dtype=el, device=DEV), torch.zeros(T, Hh, device=DEV)
        H().latent_store(d(proj), NP, Qr, Cr, R, Hh, d(wq), d(wkv), eps, d(pos), d(fq), mag, rd, d(slots), cq, cache, gate, T, f32)
        out = torch.zeros(T, Hh * Cr, dtype=el, device=DEV)
        tables = torch.stack([bt[s] for s, _, _ in parts])
        H().latent_attn(d(qa), d(q), cache, gate, d(tables), mb, d(pos), len(parts), T, Hh, D, R, Cr, bs, win, scale, d(fq), mag, rd, out,
                        f32, cu_q=d(cu), q_abs_elem=mfma, workspace=ws)
        return cq, out

    n0, n1 = lens
    cut = n1 * 2 // 5 + 1
    cq1, o1 = launch([(0, 0, n0), (1, 0, cut)])
    cq2, o2 = launch([(1, cut, n1 - 3)])
    o3 = [launch([(1, t, t + 1)])[1] for t in range(n1 - 3, n1)]             # single rows: the key-slice form where it applies
    got = {0: o1[:n0], 1: torch.cat([o1[n0:], o2] + o3)}
    for s, n in enumerate(lens):
        pr = proj_all[s].double()
        c = Z.rms(pr[:, Qr:Qr + Cr], wkv.double(), eps)
        pos = torch.arange(n)
        kr = Z.rope(pr[:, Qr + Cr:Qr + Cr + R], pos, freqs, mag, rd)
        if not f32:
            c, kr = c.bfloat16().double(), kr.bfloat16().double()
        qr = Z.rope(q_all[s].double().view(n, Hh, D + R)[..., D:], pos, freqs, mag, rd)
        sc = (torch.einsum("ihc,jc->hij", qabs_all[s].double().view(n, Hh, Cr), c) + torch.einsum("ihr,jr->hij", qr, kr)) * scale
        dist = pos[:, None] - pos[None, :]
        seen = (dist >= 0) & ((dist < win) if win else (dist >= 0))
        p = torch.softmax(sc.masked_fill(~seen[None], float("-inf")), -1)
        ref = torch.einsum("hij,jc->ihc", p, c) * torch.sigmoid(pr[:, Qr + Cr + R:])[..., None]
        assert torch.allclose(got[s].cpu().double().view(n, Hh, Cr), ref, **tol(f32)), s
    ref_cq = Z.rms(proj_all[0][:, :Qr].double(), wq.double(), eps)
    assert torch.allclose(cq1[:n0].cpu().double(), ref_cq, **tol(f32))


@pytest.mark.parametrize("Hh,D,Dv", [(6, 32, 32), (3, 16, 24), (1, 8, 1), (2, 40, 130), (2, 128, 128), (3, 64, 96), (1, 256, 32), (2, 32, 48)])
def test_lightning_scan_in_portions_over_state_slots(Hh, D, Dv):
    """Head sizes of the register form (dim 32 / 64 / 128 / 256, vdim in multiples of 32) and of the LDS form (anything else).
    Three sequences over four slots (filled with NaN: a sequence that starts at position 0 must not read its slot), fed whole, in
    portions and token by token; the state of a portion's end is what the next portion starts from."""
    lens = [29, 1, 14]
    decay = torch.tensor([math.exp(-1.0 / (1.5 ** (h + 1))) for h in range(Hh)])
    NP = 2 * Hh * D + 2 * Hh * Dv + 5
    q_off, k_off, v_off = 3, 3 + Hh * D, 3 + 2 * Hh * D
    projs = [rnd(n, NP, seed=40 + i) for i, n in enumerate(lens)]
    state = torch.full((4, Hh, D, Dv), float("nan"), device=DEV)
    d = lambda t: t.to(DEV)

    def launch(parts, slots, q_per_seq=0):
        proj = torch.cat([projs[s][lo:hi] for s, lo, hi in parts])
        pos = torch.cat([torch.arange(lo, hi) for s, lo, hi in parts])
        cu = None if q_per_seq else d(torch.tensor([0] + list(torch.tensor([hi - lo for _, lo, hi in parts]).cumsum(0)), dtype=torch.int32))
        out = torch.zeros(proj.shape[0], Hh * Dv, device=DEV)
        H().lightning_scan(d(proj), NP, q_off, k_off, v_off, d(decay), d(pos), d(torch.tensor(slots, dtype=torch.int32)), state, out,
                           len(parts), Hh, D, Dv, cu_q=cu, q_per_seq=q_per_seq)
        return out.cpu()

    refs = []
    for s, n in enumerate(lens):
        pr = projs[s].double()
        q, k, v = (Z.silu(pr[:, o:o + Hh * w]).view(n, Hh, w) for o, w in ((q_off, D), (k_off, D), (v_off, Dv)))
        S, o = torch.zeros(Hh, D, Dv, dtype=torch.float64), torch.zeros(n, Hh, Dv, dtype=torch.float64)
        for t in range(n):
            S = decay.double()[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
            o[t] = torch.einsum("hde,hd->he", S, q[t])
        refs.append(o.reshape(n, Hh * Dv))
    whole = launch([(0, 0, 29), (1, 0, 1), (2, 0, 14)], [3, 0, 1])
    assert torch.allclose(whole.double(), torch.cat(refs), rtol=1e-4, atol=1e-4)
    a = launch([(0, 0, 11), (2, 0, 2)], [2, 0])
    b = launch([(2, 2, 14), (0, 11, 12)], [0, 2])
    c = launch([(0, 12, 29)], [2])
    parts = torch.cat([a[:11], b[12:], c, whole[29:30], a[11:], b[:12]])
    assert torch.equal(parts, whole)
    outs = [launch([(0, 0, 1), (2, 0, 1)], [1, 3], q_per_seq=1)]
    for t in range(1, 14):
        outs.append(launch([(0, t, t + 1), (2, t, t + 1)], [1, 3], q_per_seq=1))
    assert torch.equal(torch.stack([o[0] for o in outs]), whole[:14]) and torch.equal(torch.stack([o[1] for o in outs]), whole[30:])


@pytest.mark.parametrize("f32", [True, False])
def test_lightning_gate_norm(f32):
    el = elem(f32)
    T, N, ld, off = 6, 136, 300, 150
    o, proj, w = rnd(T, N, seed=1, scale=3.0), rnd(T, ld, seed=2), (1 + 0.1 * rnd(N, seed=3)).to(el)
    out = torch.zeros(T, N, dtype=el, device=DEV)
    H().lightning_gate_norm(o.to(DEV), proj.to(DEV), ld, off, w.to(DEV), 1e-5, out, T, N, f32)
    ref = Z.rms(o.double(), w.double(), 1e-5) * torch.sigmoid(proj[:, off:off + N].double())
    assert torch.allclose(out.cpu().double(), ref, **tol(f32))
