"""The Zerusun decoder on MI355X: PARALLEL layers (mixer and feed-forward read one Dynamic-Tanh-normed row, their sum joins an fp32
residual), two kinds of mixer -- latent attention with a sliding window over a paged cache, and linear attention with per-head decay
over a recurrent fp32 state kept in per-sequence slots -- dense (tanh-gelu GLU) or routed (softmax router with group-limited choice,
silu GLU experts, gated shared expert) feed-forwards, and a span of layers that runs several passes with the same weights, each pass
entered through x <- W_in [x; x0] + step[pass].

Launches per layer run (T token rows):
    latent attention   [dq | dkv | gate] GEMM -> latent_store (norms, rope, cache row, gates) -> W_uq GEMM -> per-head W_uk^T GEMM
                       (queries into the latent space) -> latent_attn -> per-head W_uv GEMM -> W_o GEMM
    linear attention   [q | k | v | g] GEMM -> lightning_scan (state slot) -> lightning_gate_norm -> W_o GEMM
    dense ff           [gate | up] GEMM with the GLU as epilogue (fp32 mode: + glu_rows) -> down GEMM
    routed ff          [router | shared gate] GEMM -> moe_route_softmax -> moe_plan -> grouped [gate | up] GEMM (GLU epilogue) ->
                       grouped down GEMM -> shared [gate | up] GEMM (GLU epilogue) -> shared down GEMM
    parallel_tail      x += mixer + ff (the routed mix rides along) and the next layer's norm, or the [x | x0] row of a loop entry
over pre-allocated buffers (nothing is allocated during a forward).  Same interface as ssd_amd.model.HipDecoder towards the ModelRunner.

Arithmetic: residual rows, norms, rope angles, scores, softmax, router, recurrent state, gates and every GEMM accumulator are fp32 in
both modes.  dtype "bfloat16": weights, GEMM-input rows and the latent cache are bf16; "float32": they are fp32 and products are FMA chains.
"""
from __future__ import annotations

import torch

from ssd_amd.hip import ops as H
from ssd_amd.model import AttnMeta
from ssd_amd.model_config import ZerusunConfig
from ssd_amd.res32 import Res32Decoder

BF16 = torch.bfloat16


class HipZerusun(Res32Decoder):
    def __init__(self, cfg: ZerusunConfig, *, max_tokens: int, max_seqs: int, max_blocks: int, block_size: int, max_model_len: int,
                 device: torch.device, tp_rank: int = 0, tp_size: int = 1, tp_group=None, max_logit_rows: int | None = None,
                 max_split_tokens: int = 256, force_collectives: bool = False, taps=None, dtype: str = "bfloat16"):
        assert tp_size == 1 and taps is None, "Zerusun models are single-rank and have no activation taps"
        assert dtype in ("bfloat16", "float32")
        self.cfg, self.device = cfg, device
        self.f32 = dtype == "float32"
        self.elem = torch.float32 if self.f32 else BF16
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.use_coll, self.custom_ar, self.acts = False, None, None
        self.h = self.W = cfg.hidden_size
        self.V = cfg.vocab_size
        self.Vp = -(-self.V // 8) * 8
        self.block_size, self.max_blocks = block_size, max_blocks
        self.max_tokens = max_tokens
        self.max_logit_rows = max_logit_rows or max_tokens
        self.runs = cfg.runs()
        self.state_slots = max_seqs if cfg.recurrent else 0      # one per live sequence; the block manager hands them out
        self.w: dict[str, torch.Tensor] = {}
        self.kv: list[torch.Tensor | None] = []
        self.state: list[torch.Tensor | None] = []
        self.rope: dict[int, tuple[torch.Tensor, float]] = {}
        self.tap_residuals: list | None = None         # tests: receives a copy of the residual rows after every layer run (eager only)

        def z(*shape, dtype=torch.float32):
            return torch.zeros(*shape, dtype=dtype, device=device)

        T, W, el = max_tokens, self.W, self.elem
        lat = [l.mixer for l in cfg.layers if l.mixer.kind == "latent_attention"]
        lin = [l.mixer for l in cfg.layers if l.mixer.kind == "lightning"]
        dense = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "dense"]
        moes = [l.mlp for l in cfg.layers if l.mlp is not None and l.mlp.kind == "moe"]
        self.x = z(T, W)
        self.x0 = z(T, W) if cfg.has_loop else None
        self.cat = z(T * 2 * W, dtype=el) if cfg.has_loop else None          # rows [x | x0] of a loop entry
        self.hn = z(T, W, dtype=el)
        self.y_mix = z(T, W)
        self.y_ff = z(T, W) if dense else None
        self.proj = z(T * max([self._nproj(m) for m in lat + lin]))
        self.att = z(T * max(m.heads * m.vdim for m in lat + lin), dtype=el)
        if lat:
            self.cq = z(T * max(m.q_rank for m in lat), dtype=el)
            self.q = z(T * max(m.heads * (m.dim + m.rot_dim) for m in lat), dtype=el)
            self.q_abs = z(T * max(m.heads * m.kv_rank for m in lat))           # queries in the latent space: fp32, or (its first half)
            self.q_lat = self.q_abs.view(el)                                     # element-type rows where the MFMA attention takes them
            self.mfma = {i: H.latent_attn_mfma_ok(l.mixer.kv_rank, l.mixer.rot_dim, self.f32) for i, l in enumerate(cfg.layers)
                         if l.mixer.kind == "latent_attention"}
            self.gate = z(T * max(m.heads for m in lat))
            self.olat = z(T * max(m.heads * m.kv_rank for m in lat), dtype=el)
            # key-slice partials of the decode attention (csrc/attention_latent.hip): up to 1024 (token, 16 heads, slice) units
            self.att_ws = z(1024 * (max(m.kv_rank for m in lat) * 16 + 32)) if any(self.mfma.values()) else None
        if lin:
            self.o = z(T * max(m.heads * m.vdim for m in lin))
        ffs = [2 * m.ff for m in dense] + [2 * m.top * m.ff for m in moes] + [2 * m.shared_ff for m in moes]
        if ffs:
            self.ab = z(T * max(ffs)) if self.f32 else None                   # fp32 [gate | up] rows (bf16: the GEMM epilogue applies the GLU)
            self.act = z(T * max(ffs) // 2, dtype=el)
        if moes:
            top = max(m.top for m in moes)
            self.r_z = z(T * (max(m.experts for m in moes) + 1))
            self.r_idx = z(T * top, dtype=torch.int32)
            self.r_wt = z(T * top)
            self.r_off = z(max(m.experts for m in moes) + 1, dtype=torch.int32)
            self.r_perm = z(T * top, dtype=torch.int32)
            self.r_inv = z(T * top, dtype=torch.int32)
            self.ydn = z(T * top * W)
            self.ysh = z(T, W) if any(m.shared_ff for m in moes) else None
        R = self.max_logit_rows
        self.lastn = z(R, W, dtype=el)
        self.logits32 = z(R, self.V)
        self.logits = z(R, self.Vp, dtype=BF16)

    @staticmethod
    def _nproj(m) -> int:
        if m.kind == "latent_attention":
            return m.q_rank + m.kv_rank + m.rot_dim + m.heads
        return 2 * m.heads * m.dim + 2 * m.heads * m.vdim

    # ---------------------------------------------------------------------------------------------
    def load_weights(self, weight_iter) -> None:
        """Consumes (name, tensor) pairs under the checkpoint's names.  Matrices that read the same rows are stacked ([dq | dkv | g],
        [q | k | v | g], [gate | up], [router | shared gate]), the experts' matrices into [E][2 ff][W] / [E][W][ff], W_uk per head
        transposed ([H][kv_rank][dim]: the product that carries queries into the latent space); a norm's alpha becomes one fp32 number
        in device memory."""
        raw = {n: t.to(self.device) for n, t in weight_iter}
        cv = lambda t: t.to(self.elem).contiguous()
        w = self.w = {}

        def norm(n):
            w[n], w[n + ".b"] = cv(raw[n]), cv(raw[n + ".b"])
            w[n + ".alpha"] = raw[n + ".alpha"].float().reshape(1).contiguous()

        def pair(gate, up):
            # bf16: rows interleaved (gate_0, up_0, gate_1, ...) for the GEMM's paired epilogue; fp32: [gate | up], a GLU launch follows
            return torch.stack([gate, up], dim=1).reshape(-1, gate.shape[1]) if not self.f32 else torch.cat([gate, up], dim=0)

        def glu(dst, src):
            w[dst + "gu"] = cv(pair(raw[src + "gate"], raw[src + "up"]))
            w[dst + "down"] = cv(raw[src + "down"])

        w["embed"] = cv(raw["embed"])
        norm("embed.norm")
        norm("final.norm")
        if self.cfg.has_loop:
            w["loop.in"], w["loop.step"] = cv(raw["loop.in"]), cv(raw["loop.step"])
        for i, lc in enumerate(self.cfg.layers):
            p, m, ml = f"l{i}.", lc.mixer, lc.mlp
            norm(p + "norm1")
            if m.kind == "latent_attention":
                w[p + "mix.in"] = cv(torch.cat([raw[p + "mix.dq"], raw[p + "mix.dkv"], raw[p + "mix.g"]], dim=0))
                w[p + "mix.ukt"] = cv(raw[p + "mix.uk"].view(m.heads, m.dim, m.kv_rank).transpose(1, 2))
                for n in ("mix.dq.norm", "mix.dkv.norm", "mix.uq", "mix.uv", "mix.o"):
                    w[p + n] = cv(raw[p + n])
                f, mag = m.rope.frequencies()
                self.rope[i] = (torch.tensor(f, dtype=torch.float64).to(torch.float32).to(self.device), float(mag))
            else:
                w[p + "mix.in"] = cv(torch.cat([raw[p + "mix.q"], raw[p + "mix.k"], raw[p + "mix.v"], raw[p + "mix.g"]], dim=0))
                w[p + "mix.norm"], w[p + "mix.o"] = cv(raw[p + "mix.norm"]), cv(raw[p + "mix.o"])
                w[p + "mix.decay"] = torch.tensor(m.decay, dtype=torch.float64).to(torch.float32).to(self.device)
            if ml is None:
                continue
            if ml.kind == "dense":
                glu(p + "mlp.", p + "mlp.")
                continue
            w[p + "mlp.gu"] = cv(torch.stack([pair(raw[p + f"mlp.e{e}.gate"], raw[p + f"mlp.e{e}.up"]) for e in range(ml.experts)]))
            w[p + "mlp.down"] = cv(torch.stack([raw[p + f"mlp.e{e}.down"] for e in range(ml.experts)]))
            if ml.shared_ff:
                w[p + "mlp.router"] = cv(torch.cat([raw[p + "mlp.router"], raw[p + "mlp.shared.sg"].reshape(1, -1)], dim=0))
                glu(p + "mlp.shared.", p + "mlp.shared.")
            else:
                w[p + "mlp.router"] = cv(raw[p + "mlp.router"])
        torch.cuda.synchronize(self.device)

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in self.w.values())

    def active_weight_bytes(self, T: int = 1) -> int:
        """HBM bytes of weights one forward of T tokens must stream at least: every dense matrix once per layer RUN, of the experts
        min(E, T * top) per layer run, the embedding table once as the LM head."""
        per = {n: t.numel() * t.element_size() for n, t in self.w.items()}
        total = per["embed"]
        if self.cfg.has_loop:
            total += per["loop.in"] * self.cfg.loop_times
        for li, _ in self.runs:
            p, ml = f"l{li}.", self.cfg.layers[li].mlp
            total += sum(v for n, v in per.items() if n.startswith(p + "mix.") or n.startswith(p + "norm1"))
            if ml is None:
                continue
            if ml.kind == "dense":
                total += per[p + "mlp.gu"] + per[p + "mlp.down"]
                continue
            frac = min(ml.experts, T * ml.top) / ml.experts
            total += int((per[p + "mlp.gu"] + per[p + "mlp.down"]) * frac) + per[p + "mlp.router"]
            if ml.shared_ff:
                total += per[p + "mlp.shared.gu"] + per[p + "mlp.shared.down"]
        return total

    def kv_block_bytes(self) -> int:
        es = 4 if self.f32 else 2
        n = sum((self.cfg.layers[li].mixer.kv_rank + self.cfg.layers[li].mixer.rot_dim) * self.block_size * es
                for li, _ in self.runs if self.cfg.layers[li].mixer.kind == "latent_attention")
        return max(n, 1)

    def state_bytes(self) -> int:
        """Bytes of recurrent state one live sequence holds (all layer runs)."""
        return sum(self.cfg.layers[li].mixer.heads * self.cfg.layers[li].mixer.dim * self.cfg.layers[li].mixer.vdim * 4
                   for li, _ in self.runs if self.cfg.layers[li].mixer.kind == "lightning")

    def alloc_kv(self, num_blocks: int) -> None:
        """Per layer run: a latent-attention run gets cache rows [blocks * block_size][kv_rank + rot_dim] (the latent and the rotated key
        part, for all heads together), a linear-attention run gets state [slots][H][dim][vdim] fp32.  A slot is not cleared when it is
        handed out: a forward whose rows start at position 0 starts from zero by itself."""
        self.num_blocks = num_blocks
        self.kv, self.state = [], []
        for li, _ in self.runs:
            m = self.cfg.layers[li].mixer
            if m.kind == "latent_attention":
                self.kv.append(torch.zeros(num_blocks * self.block_size, m.kv_rank + m.rot_dim, dtype=self.elem, device=self.device))
                self.state.append(None)
            else:
                self.kv.append(None)
                self.state.append(torch.zeros(self.state_slots, m.heads, m.dim, m.vdim, dtype=torch.float32, device=self.device))

    # ---------------------------------------------------------------------------------------------
    def launch_mixer(self, run: int, li: int, T: int, positions, meta: AttnMeta) -> None:
        """hn (normalised rows) -> y_mix (fp32 mixer output rows)."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        m, p = cfg.layers[li].mixer, f"l{li}.mix."
        NP = self._nproj(m)
        seqs = dict(cu_q=meta.cu_q) if meta.cu_q is not None else dict(q_per_seq=meta.q_per_seq)
        H.gemm_rows(self.hn, w[p + "in"], self.proj, T, NP, W, f)
        if m.kind == "latent_attention":
            Hh, D, R, Cr = m.heads, m.dim, m.rot_dim, m.kv_rank
            freqs, mag = self.rope[li]
            H.latent_store(self.proj, NP, m.q_rank, Cr, R, Hh, w[p + "dq.norm"], w[p + "dkv.norm"], cfg.rms_norm_eps, positions, freqs,
                           mag, m.rope.dims, meta.slot_mapping, self.cq, self.kv[run], self.gate, T, f)
            H.gemm_rows(self.cq, w[p + "uq"], self.q, T, Hh * (D + R), m.q_rank, f, H.GR_ELEM)
            mf = self.mfma[li]
            H.gemm_rows_batched(self.q, w[p + "ukt"], self.q_lat if mf else self.q_abs, T, Cr, D, Hh, Hh * (D + R), D + R, Hh * Cr, Cr, f,
                                H.GR_ELEM if mf else H.GR_F32)
            H.latent_attn(self.q_lat if mf else self.q_abs, self.q, self.kv[run], self.gate, meta.block_tables, self.max_blocks, positions,
                          meta.B, T, Hh, D, R, Cr, self.block_size, m.window, m.scale, freqs, mag, m.rope.dims, self.olat, f,
                          q_abs_elem=mf, workspace=self.att_ws, **seqs)
            H.gemm_rows_batched(self.olat, w[p + "uv"], self.att, T, m.vdim, Cr, Hh, Hh * Cr, Cr, Hh * m.vdim, m.vdim, f, H.GR_ELEM)
        else:
            Hh, D, Dv = m.heads, m.dim, m.vdim
            assert meta.state_slots is not None, "a model with recurrent layers needs the sequences' state slots"
            H.lightning_scan(self.proj, NP, 0, Hh * D, 2 * Hh * D, w[p + "decay"], positions, meta.state_slots, self.state[run], self.o,
                             meta.B, Hh, D, Dv, **seqs)
            H.lightning_gate_norm(self.o, self.proj, NP, 2 * Hh * D + Hh * Dv, w[p + "norm"], cfg.rms_norm_eps, self.att, T, Hh * Dv, f)
        H.gemm_rows(self.att, w[p + "o"], self.y_mix, T, W, m.heads * m.vdim, f)

    def launch_mlp(self, li: int, T: int) -> dict:
        """hn -> the feed-forward's rows; returns the keyword arguments that hand them to parallel_tail."""
        w, f, W = self.w, self.f32, self.W
        ml, p = self.cfg.layers[li].mlp, f"l{li}.mlp."
        if ml is None:
            return {}
        if ml.kind == "dense":
            self._glu_gemm(self.hn, w[p + "gu"], T, ml.ff, H.GLU_GELU_TANH)
            H.gemm_rows(self.act, w[p + "down"], self.y_ff, T, W, ml.ff, f)
            return dict(y_ff=self.y_ff)
        E, top = ml.experts, ml.top
        ldz = E + (1 if ml.shared_ff else 0)
        H.gemm_rows(self.hn, w[p + "router"], self.r_z, T, ldz, W, f)
        H.moe_route_softmax(self.r_z, ldz, self.r_idx, self.r_wt, T, E, top, ml.groups, ml.keep, ml.scale)
        H.moe_plan(self.r_idx, T, top, E, self.r_off, self.r_perm, self.r_inv)
        if f:
            H.gemm_rows_grouped(self.hn, w[p + "gu"], self.ab, self.r_off, E, T * top, 2 * ml.ff, W, f, H.GR_F32, row_idx=self.r_perm,
                                idx_div=top)
            H.glu_rows(self.ab, self.act, T * top, ml.ff, H.GLU_SILU, f)
        else:
            H.gemm_rows_grouped(self.hn, w[p + "gu"], self.act, self.r_off, E, T * top, 2 * ml.ff, W, f, H.GR_GLU_SILU, row_idx=self.r_perm,
                                idx_div=top)
        H.gemm_rows_grouped(self.act, w[p + "down"], self.ydn, self.r_off, E, T * top, W, ml.ff, f, H.GR_F32)
        out = dict(ydn=self.ydn, inv=self.r_inv, weights=self.r_wt, top=top)
        if ml.shared_ff:
            self._glu_gemm(self.hn, w[p + "shared.gu"], T, ml.shared_ff, H.GLU_SILU)
            H.gemm_rows(self.act, w[p + "shared.down"], self.ysh, T, W, ml.shared_ff, f)
            out.update(shared=self.ysh, shared_gate=self.r_z.view(-1)[E:], ld_shared_gate=ldz)
        return out

    def _glu_gemm(self, x, w_gu, T: int, ff: int, act: int) -> None:
        """self.act = act(W_gate x) * (W_up x): in bf16 the GEMM's paired epilogue (weight rows interleaved at load), in fp32 a
        [gate | up] GEMM with fp32 rows out and the GLU launch."""
        if self.f32:
            H.gemm_rows(x, w_gu, self.ab, T, 2 * ff, self.W, True)
            H.glu_rows(self.ab, self.act, T, ff, act, True)
        else:
            H.gemm_rows(x, w_gu, self.act, T, 2 * ff, self.W, False, H.GR_GLU_SILU if act == H.GLU_SILU else H.GR_GLU_GELU)

    def _enters_pass(self, run: int) -> bool:
        return self.cfg.has_loop and self.runs[run][0] == self.cfg.loop_start

    def _loop_entry(self, run: int, T: int) -> None:
        """cat = [x | x0] rows -> x = W_in cat + step[pass]; hn = the entered layer's norm of x."""
        w, W = self.w, self.W
        li, ps = self.runs[run]
        H.gemm_rows(self.cat, w["loop.in"], self.x, T, W, 2 * W, self.f32)
        n = f"l{li}.norm1"
        H.dyt_rows(self.x, w[n + ".alpha"], w[n], w[n + ".b"], self.hn, T, W, self.f32, add_vec=w["loop.step"][ps])

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, T: int, meta: AttnMeta) -> None:
        """Runs every layer run over the T token rows; leaves the fp32 residual rows in self.x."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        assert T <= self.max_tokens and meta.mode == H.MODE_CAUSAL and (meta.cu_q is not None or meta.q_per_seq > 0)
        fuse = self.tap_residuals is None
        norm = lambda n: dict(next_alpha=w[n + ".alpha"], next_weight=w[n], next_bias=w[n + ".b"], next_out=self.hn)
        e = "embed.norm"
        right = self.cat[W:] if cfg.has_loop else None
        H.dyt_embed(input_ids, w["embed"], w[e + ".alpha"], w[e], w[e + ".b"], self.x, self.x0, right, 2 * W, T, W, f)
        if self._enters_pass(0):       # the loop starts at the first layer: the left half of [x | x0] is the embedding output too
            H.dyt_embed(input_ids, w["embed"], w[e + ".alpha"], w[e], w[e + ".b"], self.x, None, self.cat, 2 * W, T, W, f)
        for run, (li, ps) in enumerate(self.runs):
            if self._enters_pass(run):
                self._loop_entry(run, T)
            elif run == 0 or not fuse:
                n = f"l{li}.norm1"
                H.dyt_rows(self.x, w[n + ".alpha"], w[n], w[n + ".b"], self.hn, T, W, f)
            self.launch_mixer(run, li, T, positions, meta)
            ff = self.launch_mlp(li, T)
            nxt = {}
            if run + 1 < len(self.runs):
                if self._enters_pass(run + 1):
                    nxt = dict(cat=self.cat, ld_cat=2 * W)
                elif fuse:
                    nxt = norm(f"l{self.runs[run + 1][0]}.norm1")
            H.parallel_tail(self.x, self.y_mix, T, W, f, **ff, **nxt)
            if not fuse:
                self.tap_residuals.append(self.x[:T].clone())

    def compute_logits(self, T: int, gather: torch.Tensor | None = None, rows: int | None = None) -> int:
        """Final norm (optionally of the `gather` rows only) and the LM head = the embedding table: fp32 logits in logits32[:n], their
        bf16 rounding (row stride Vp, padding -inf) in logits[:n] for the sampling kernels.  Returns n."""
        n = T if gather is None else rows
        assert n <= self.max_logit_rows
        w, e = self.w, "final.norm"
        H.dyt_rows(self.x, w[e + ".alpha"], w[e], w[e + ".b"], self.lastn, n, self.W, self.f32, gather=gather)
        H.gemm_rows(self.lastn, w["embed"], self.logits32, n, self.V, self.W, self.f32)
        H.rows_f32_to_bf16(self.logits32, self.logits, n, self.V, self.V, self.Vp)
        return n
