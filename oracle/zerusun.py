"""Plain whole-sequence statement of the Zerusun decoder, one function per mechanism, in float64 on the CPU.

No cache, no state slots, no batching: a sequence is a [T] token list and every function sees all of its rows at once (the recurrent
mixer is a literal loop over the tokens).  Shares no code with ssd_amd/; the tests compare the engine against it.

Notation: W = model width, x = fp residual rows [T, W], h = normalised rows, P[name] = the checkpoint tensor of that name as float64.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def dyt(x, w, b, alpha):
    """Dynamic Tanh: tanh(alpha x) * w + b (no statistics of x)."""
    return torch.tanh(alpha * x) * w + b


def rms(x, w, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def rope_frequencies(dims: int, base: float, scaling: dict | None):
    """Per-pair angular frequencies f_i (i < dims / 2) and the factor both cos and sin carry.  YaRN: pairs that turn fast keep their
    frequency, pairs that turn slowly are slowed by `factor`, a linear ramp between the two corner pairs."""
    half = dims // 2
    i = torch.arange(half, dtype=F64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])

    def corner(turns):
        return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))
    lo = max(math.floor(corner(float(scaling["fast"]))), 0)
    hi = min(math.ceil(corner(float(scaling["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rope(x, pos, freqs, mag, dims: int):
    """x [T, ..., n]: the first `dims` entries of the last axis rotate (entry i pairs with i + dims / 2), the rest pass."""
    half = dims // 2
    ang = pos.to(F64)[:, None] * freqs[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = (torch.cos(ang) * mag).reshape(shape), (torch.sin(ang) * mag).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def latent_attention(h, P, p, m, eps):
    """Queries and keys / values through low-rank latents; one rotated key part shared by all heads; sliding window; per-head
    sigmoid output gate.  m: the layer's mixer dict of config.json."""
    T = h.shape[0]
    Hh, D, R, Dv, kvr = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    rot = m["rot"]
    freqs, mag = rope_frequencies(rot["dims"], float(rot["base"]), rot.get("scaling"))
    cq = rms(h @ P[p + "dq"].T, P[p + "dq.norm"], eps)
    q = (cq @ P[p + "uq"].T).view(T, Hh, D + R)
    q_nope, q_rot = q[..., :D], rope(q[..., D:], pos, freqs, mag, rot["dims"])
    dkv = h @ P[p + "dkv"].T
    c = rms(dkv[:, :kvr], P[p + "dkv.norm"], eps)
    k_rot = rope(dkv[:, kvr:], pos, freqs, mag, rot["dims"])                 # [T, R], the same for every head
    k_nope = (c @ P[p + "uk"].T).view(T, Hh, D)
    v = (c @ P[p + "uv"].T).view(T, Hh, Dv)
    s = (torch.einsum("ihd,jhd->hij", q_nope, k_nope) + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * float(m["scale"])
    win = (m.get("mask") or {}).get("size")
    dist = pos[:, None] - pos[None, :]
    seen = (dist >= 0) & ((dist < win) if win else (dist >= 0))
    s = s.masked_fill(~seen[None], float("-inf"))
    o = torch.einsum("hij,jhd->ihd", torch.softmax(s, dim=-1), v)
    gate = torch.sigmoid(h @ P[p + "g"].T)                                   # [T, heads]
    return (o * gate[..., None]).reshape(T, Hh * Dv) @ P[p + "o"].T


def lightning(h, P, p, m, eps):
    """Linear attention with a per-head scalar decay: S <- decay S + k v^T, o = S^T q, token by token from S = 0."""
    T = h.shape[0]
    Hh, D, Dv = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ P[p + "q"].T).view(T, Hh, D)
    k = silu(h @ P[p + "k"].T).view(T, Hh, D)
    v = silu(h @ P[p + "v"].T).view(T, Hh, Dv)
    decay = torch.tensor(m["decay"], dtype=F64)
    S = torch.zeros(Hh, D, Dv, dtype=F64)
    o = torch.zeros(T, Hh, Dv, dtype=F64)
    for t in range(T):
        S = decay[:, None, None] * S + k[t][:, :, None] * v[t][:, None, :]
        o[t] = torch.einsum("hde,hd->he", S, q[t])
    o = rms(o.reshape(T, Hh * Dv), P[p + "norm"], eps) * torch.sigmoid(h @ P[p + "g"].T)
    return o @ P[p + "o"].T


def glu(h, P, p, act):
    return (act(h @ P[p + "gate"].T) * (h @ P[p + "up"].T)) @ P[p + "down"].T


def route(z, r):
    """Router logits z [T, E] -> (chosen experts [T, top], their weights): softmax over all experts, experts outside the best
    groups dropped, the top scores kept, renormalised and scaled."""
    s = torch.softmax(z, dim=-1)
    T, E = s.shape
    g = r.get("groups") or {"count": 1, "keep": 1}
    per = E // g["count"]
    best = s.view(T, g["count"], per).max(dim=-1).values.topk(g["keep"], dim=-1).indices
    allowed = torch.zeros(T, g["count"], dtype=torch.bool).scatter_(1, best, True).repeat_interleave(per, dim=1)
    idx = s.masked_fill(~allowed, -1.0).topk(r["top"], dim=-1).indices
    wt = s.gather(1, idx)
    return idx, wt / (wt.sum(dim=-1, keepdim=True) + 1e-20) * float(r["scale"])


def moe(h, P, p, ml):
    idx, wt = route(h @ P[p + "router"].T, ml["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, w in zip(idx[t].tolist(), wt[t]):
            out[t] += w * glu(h[t:t + 1], P, p + f"e{e}.", silu)[0]
    if ml.get("shared"):
        out = out + torch.sigmoid(h @ P[p + "shared.sg"].T) * glu(h, P, p + "shared.", silu)
    return out


def feed_forward(h, P, p, ml):
    if ml is None:
        return torch.zeros_like(h)
    return glu(h, P, p, gelu_tanh) if ml["kind"] == "dense" else moe(h, P, p, ml)


def layer_runs(cfg) -> list[tuple[int, int, bool]]:
    """(layer, pass, first of its pass) for every layer run."""
    n, lp = len(cfg["layers"]), cfg.get("loop") or {}
    a, b, times = lp.get("start", 0), lp.get("stop", 0), lp.get("times", 1)
    if b <= a:
        return [(i, 0, False) for i in range(n)]
    span = [(i, t, i == a) for t in range(times) for i in range(a, b)]
    return [(i, 0, False) for i in range(a)] + span + [(i, 0, False) for i in range(b, n)]


def forward(cfg: dict, weights: dict, tokens, taps: list | None = None):
    """Logits [T, vocab] of one sequence; taps receives the residual rows after every layer run."""
    P = {n: t.to(F64) for n, t in weights.items()}
    eps = float(cfg["norm"]["eps"])
    norm = lambda x, n: dyt(x, P[n], P[n + ".b"], P[n + ".alpha"])
    x = norm(P["embed"][torch.as_tensor(tokens)], "embed.norm")
    x0 = x
    for li, t, first in layer_runs(cfg):
        lc, p = cfg["layers"][li], f"l{li}."
        if first:
            x = torch.cat([x, x0], dim=-1) @ P["loop.in"].T + P["loop.step"][t]
        h = norm(x, p + "norm1")
        mixer = {"latent_attention": latent_attention, "lightning": lightning}[lc["type"]]
        x = x + (mixer(h, P, p + "mix.", lc["mixer"], eps) + feed_forward(h, P, p + "mlp.", lc.get("mlp")))
        if taps is not None:
            taps.append(x.clone())
    return norm(x, "final.norm") @ P["embed"].T


# ---------------------------------------------------------------------------------------------------------------------
# small self-made models for the tests
# ---------------------------------------------------------------------------------------------------------------------
def latent_layer(heads=4, dim=16, rot_dim=8, vdim=24, q_rank=40, kv_rank=48, window=9, scale=None, rot_dims=None, base=10000.0,
                 scaling="yarn", mlp=None) -> dict:
    sc = {"factor": 4.0, "original": 64, "fast": 32.0, "slow": 1.0} if scaling == "yarn" else scaling
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
                      "scale": scale if scale is not None else (dim + rot_dim) ** -0.5, "mask": {"size": window} if window else None,
                      "rot": {"dims": rot_dims or rot_dim, "base": base, "scaling": sc}}}


def lightning_layer(heads=3, dim=16, vdim=24, decay=None, mlp=None) -> dict:
    decay = decay or [math.exp(-1.0 / (2.0 ** (1 + 1.5 * h))) for h in range(heads)]
    return {"type": "lightning", "mlp": mlp, "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": decay}}


def dense_mlp(ff=40) -> dict:
    return {"kind": "dense", "ff": ff}


def moe_mlp(experts=8, top=2, ff=24, groups=(2, 1), scale=1.5, shared_ff=40) -> dict:
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "top": top, "scale": scale, "groups": {"count": groups[0], "keep": groups[1]} if groups else None},
            "shared": {"ff": shared_ff} if shared_ff else None}


def make_config(layers, vocab=96, width=64, loop=(0, 0, 1), eps=1e-5) -> dict:
    return {"architecture": "Zerusun", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers,
            "loop": {"start": loop[0], "stop": loop[1], "times": loop[2]}}


def random_model(cfg: dict, seed: int = 0) -> dict:
    """bf16 weights of the right shapes for `cfg`: matrices N(0, 1 / fan-in) (queries a little sharper), norm weights around 1."""
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def mat(name, o, i, gain=1.0):
        w[name] = (torch.randn(o, i, generator=gen) * gain / math.sqrt(i)).to(torch.bfloat16)

    def vec(name, n, base=1.0, s=0.1):
        w[name] = (base + s * torch.randn(n, generator=gen)).to(torch.bfloat16)

    def norm(name):
        vec(name, W)
        vec(name + ".b", W, 0.0, 0.1)
        w[name + ".alpha"] = torch.tensor(0.4 + 0.4 * torch.rand((), generator=gen).item()).to(torch.bfloat16)

    def glu_w(p, ff):
        mat(p + "gate", ff, W, 1.5)
        mat(p + "up", ff, W, 1.5)
        mat(p + "down", W, ff)

    mat("embed", cfg["vocab"], W, math.sqrt(W))
    norm("embed.norm")
    norm("final.norm")
    lp = cfg.get("loop") or {}
    if lp.get("stop", 0) > lp.get("start", 0):
        mat("loop.in", W, 2 * W, 1.2)
        w["loop.step"] = (0.3 * torch.randn(lp["times"], W, generator=gen)).to(torch.bfloat16)
    for i, lc in enumerate(cfg["layers"]):
        p, m = f"l{i}.", lc["mixer"]
        norm(p + "norm1")
        Hh = m["heads"]
        if lc["type"] == "latent_attention":
            mat(p + "mix.dq", m["q_rank"], W)
            vec(p + "mix.dq.norm", m["q_rank"])
            mat(p + "mix.uq", Hh * (m["dim"] + m["rot_dim"]), m["q_rank"], 3.0)
            mat(p + "mix.dkv", m["kv_rank"] + m["rot_dim"], W, 1.5)
            vec(p + "mix.dkv.norm", m["kv_rank"])
            mat(p + "mix.uk", Hh * m["dim"], m["kv_rank"], 1.5)
            mat(p + "mix.uv", Hh * m["vdim"], m["kv_rank"])
            mat(p + "mix.g", Hh, W)
        else:
            for n, d in (("q", m["dim"]), ("k", m["dim"]), ("v", m["vdim"]), ("g", m["vdim"])):
                mat(p + "mix." + n, Hh * d, W, 1.5)
            vec(p + "mix.norm", Hh * m["vdim"])
        mat(p + "mix.o", W, Hh * m["vdim"])
        ml = lc.get("mlp")
        if ml is None:
            continue
        if ml["kind"] == "dense":
            glu_w(p + "mlp.", ml["ff"])
            continue
        for e in range(ml["router"]["experts"]):
            glu_w(p + f"mlp.e{e}.", ml["expert"]["ff"])
        mat(p + "mlp.router", ml["router"]["experts"], W, 2.0)
        if ml.get("shared"):
            glu_w(p + "mlp.shared.", ml["shared"]["ff"])
            mat(p + "mlp.shared.sg", 1, W)
    return w
