"""Plain, slow statement of the Fatulix decoder (TEST INFRASTRUCTURE ONLY; shares nothing with ssd_amd/).

One function per mechanism, written from the equations, on whole sequences without any cache: every position attends by a
mask over the full score matrix.  `dtype` is the arithmetic of the matrix products (float64 for a sharp reference, float32
otherwise); everything else is computed in that same type.

Notation.  E = eps of the layer.  rms(x) = x / sqrt(mean(x^2) + E) over the last axis.
  sandwich layer:       x <- x + w1b * rms(mixer(w1 * rms(x)));  x <- x + w2b * rms(ff(w2 * rms(x)))
  differential mixer:   per query head h (kv head h // (H/G)), maps m = 1, 2 over the SAME values:
                          P_m = softmax_causal(scale * rms(q_hm) wq . rms(k_gm) wk);  a_m = P_m v_g
                          L = exp(<lq1, lk1>) - exp(<lq2, lk2>) + d
                          o_h = (1 - d) * rms_noweight(a_1 - L a_2) * sigmoid(W_g x)_h
  routed feed-forward:  z = W_r x;  S = the `top` largest z;  y = sum_{e in S} softmax(z_S)_e * W_down,e relu(W_up,e x)^2 + shared(x)
  layer loop:           layers [start, stop) run `times` passes with the same weights; before every pass after the first the
                        embedding output is added to x.
"""
from __future__ import annotations

import math

import torch


def rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm(x, w, eps):
    return rms(x, eps) * w


def causal_softmax(scores: torch.Tensor) -> torch.Tensor:
    """scores [..., T, T]; row i sees columns j <= i."""
    T = scores.shape[-1]
    mask = torch.ones(T, T, dtype=torch.bool).tril()
    return torch.softmax(scores.masked_fill(~mask, float("-inf")), dim=-1)


def diff_lambda(w: dict, p: str, diff: float, dtype) -> float:
    g = lambda n: w[p + n].to(dtype)
    return float(torch.exp((g("lq1") * g("lk1")).sum()) - torch.exp((g("lq2") * g("lk2")).sum()) + diff)


def diff_attention(h: torch.Tensor, w: dict, p: str, m: dict, eps: float, dtype) -> torch.Tensor:
    """h [T, width] -> mixer output [T, width]."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    g = lambda n: w[p + n].to(dtype)
    q = (h @ g("q").T).view(T, H, 2, D)
    k = (h @ g("k").T).view(T, G, 2, D)
    v = (h @ g("v").T).view(T, G, Dv)
    q = norm(q, g("q.norm"), eps)
    k = norm(k, g("k.norm"), eps)
    lam = diff_lambda(w, p, m["diff"], dtype)
    gate = torch.sigmoid(h @ g("g").T)                      # [T, H]
    heads = []
    for hh in range(H):
        kv = hh // (H // G)
        a = []
        for mp in range(2):
            s = (q[:, hh, mp] @ k[:, kv, mp].T) * m["scale"]
            a.append(causal_softmax(s) @ v[:, kv])
        o = a[0] - lam * a[1]
        o = rms(o, eps) * (1.0 - m["diff"])
        heads.append(o * gate[:, hh:hh + 1])
    return torch.cat(heads, dim=-1) @ g("o").T


def expert(h, w_up, w_down):
    return (torch.relu(h @ w_up.T) ** 2) @ w_down.T


def route(h, w_router, top: int):
    """Indices [T, top] and weights [T, top] (softmax over the chosen logits only)."""
    z = h @ w_router.T
    val, idx = z.topk(top, dim=-1)
    return idx, torch.softmax(val, dim=-1)


def moe(h: torch.Tensor, w: dict, p: str, m: dict, dtype) -> torch.Tensor:
    g = lambda n: w[p + n].to(dtype)
    E, top = m["router"]["experts"], m["router"]["top"]
    idx, wt = route(h, g("router"), top)
    out = torch.zeros(h.shape[0], w[p + "e0.down"].shape[0], dtype=dtype)
    for t in range(h.shape[0]):
        for j in range(top):
            e = int(idx[t, j])
            assert e < E
            out[t] += wt[t, j] * expert(h[t], g(f"e{e}.up"), g(f"e{e}.down"))
    if m.get("shared"):
        out = out + expert(h, g("shared.up"), g("shared.down"))
    return out


def layer_runs(cfg: dict) -> list[tuple[int, int]]:
    """(layer index, pass index) of every layer run in execution order; pass index counts repeats of the looped span."""
    L = len(cfg["layers"])
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    a, b, n = loop["start"], loop["stop"], loop["times"]
    runs = [(i, 0) for i in range(a)]
    for ps in range(n if b > a else 0):
        runs += [(i, ps) for i in range(a, b)]
    runs += [(i, 0) for i in range(b, L)]
    return runs


def forward(cfg: dict, w: dict, tokens, dtype=torch.float64, residuals: list | None = None) -> torch.Tensor:
    """Logits [T, vocab] of one whole sequence.  residuals (optional list) receives x after every layer run."""
    eps = cfg["norm"]["eps"]
    g = lambda n: w[n].to(dtype)
    x0 = g("embed")[torch.as_tensor(tokens, dtype=torch.long)]
    x = x0.clone()
    loop = cfg.get("loop") or {"start": 0, "stop": 0, "times": 1}
    for li, ps in layer_runs(cfg):
        if ps > 0 and li == loop["start"]:
            x = x + x0
        lc, p = cfg["layers"][li], f"l{li}."
        assert lc["type"] == "attention"
        y = diff_attention(norm(x, g(p + "norm1"), eps), w, p + "mix.", lc["mixer"], eps, dtype)
        x = x + norm(y, g(p + "norm1b"), eps)
        if lc.get("mlp"):
            assert lc["mlp"]["kind"] == "moe"
            y = moe(norm(x, g(p + "norm2"), eps), w, p + "mlp.", lc["mlp"], dtype)
            x = x + norm(y, g(p + "norm2b"), eps)
        if residuals is not None:
            residuals.append(x.clone())
    return norm(x, g("final.norm"), eps) @ g("head").T


def random_model(cfg: dict, seed: int = 0, std: float = 0.5) -> dict:
    """bf16 weights of the right shapes for `cfg` (norm weights around 1)."""
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def mat(name, o, i, s=None):
        w[name] = (torch.randn(o, i, generator=gen) * (s if s is not None else std / math.sqrt(i))).to(torch.bfloat16)

    def vec(name, n, base=1.0, s=0.1):
        w[name] = (base + s * torch.randn(n, generator=gen)).to(torch.bfloat16)

    mat("embed", cfg["vocab"], W, 1.0)
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        for n in ("norm1", "norm1b") + (("norm2", "norm2b") if lc.get("mlp") else ()):
            vec(p + n, W)
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        mat(p + "mix.q", H * 2 * D, W, 2.0 / math.sqrt(W))
        mat(p + "mix.k", G * 2 * D, W, 2.0 / math.sqrt(W))
        mat(p + "mix.v", G * Dv, W)
        vec(p + "mix.q.norm", D)
        vec(p + "mix.k.norm", D)
        for n in ("lq1", "lk1", "lq2", "lk2"):
            vec(p + "mix." + n, D, 0.0, 0.2)
        mat(p + "mix.g", H, W, 1.0 / math.sqrt(W))
        mat(p + "mix.o", W, H * Dv)
        ml = lc.get("mlp")
        if ml:
            for e in range(ml["router"]["experts"]):
                mat(p + f"mlp.e{e}.up", ml["expert"]["ff"], W, 1.0 / math.sqrt(W))
                mat(p + f"mlp.e{e}.down", W, ml["expert"]["ff"])
            mat(p + "mlp.router", ml["router"]["experts"], W, 2.0 / math.sqrt(W))
            if ml.get("shared"):
                mat(p + "mlp.shared.up", ml["shared"]["ff"], W, 1.0 / math.sqrt(W))
                mat(p + "mlp.shared.down", W, ml["shared"]["ff"])
    vec("final.norm", W)
    mat("head", cfg["vocab"], W, 1.0 / math.sqrt(W))
    return w


def make_config(vocab=96, width=64, n_layers=3, heads=4, kv_heads=2, dim=16, vdim=32, diff=0.25, scale=None, experts=4, top=2,
                ff=32, shared_ff=48, loop=(0, 0, 1), eps=1e-5, no_mlp_layers=()) -> dict:
    layers = []
    for i in range(n_layers):
        mlp = None if i in no_mlp_layers else {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
                                               "shared": {"ff": shared_ff} if shared_ff else None}
        layers.append({"type": "attention", "mlp": mlp,
                       "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "diff": diff,
                                 "scale": scale if scale is not None else dim ** -0.5}})
    return {"architecture": "Fatulix", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
            "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}
