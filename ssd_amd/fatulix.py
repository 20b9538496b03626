"""The Fatulix decoder on MI355X: sandwich-normed layers over an fp32 residual stream, differential attention over a paged KV cache,
a routed (mixture-of-experts) feed-forward with a shared expert, and a span of layers that runs several passes with the same weights.

Per layer run the launch list is
    fused [q | k | v | gate] GEMM -> diffattn_store (q / k norms, KV store, gate sigmoid) -> diffattn_paged -> o GEMM ->
    sandwich_tail (post-norm + residual sum + the feed-forward's pre-norm) -> router GEMM -> moe_route -> moe_plan -> grouped up
    GEMM (relu^2 epilogue) -> grouped down GEMM -> shared up / down GEMMs -> sandwich_tail (routed mix + post-norm + residual sum +
    the embedding output before a repeated pass + the next run's pre-norm)
over pre-allocated buffers (nothing is allocated during a forward: it can be captured in a hipGraph like the other decoders).
Same interface as ssd_amd.model.HipDecoder towards the ModelRunner: forward / compute_logits / argmax / full_logits / alloc_kv.

Arithmetic: residual rows, norm statistics, q / k norms, scores, softmax weights, router logits and the expert mix are fp32 always.
dtype "bfloat16": weights, GEMM-input rows and the KV cache are bf16 (MFMA, fp32 accumulation); "float32": they are fp32 and
the products are FMA chains.  Every layer run has KV pages of its own (a repeated pass attends to ITS pass's keys).
"""
from __future__ import annotations

import torch

from ssd_amd.hip import ops as H
from ssd_amd.model import AttnMeta
from ssd_amd.model_config import FatulixConfig
from ssd_amd.res32 import Res32Decoder

BF16 = torch.bfloat16


class HipFatulix(Res32Decoder):

    def __init__(self, cfg: FatulixConfig, *, max_tokens: int, max_seqs: int, max_blocks: int, block_size: int, max_model_len: int,
                 device: torch.device, tp_rank: int = 0, tp_size: int = 1, tp_group=None, max_logit_rows: int | None = None,
                 max_split_tokens: int = 256, force_collectives: bool = False, taps=None, dtype: str = "bfloat16"):
        assert tp_size == 1 and taps is None, "Fatulix models are single-rank and have no activation taps"
        assert dtype in ("bfloat16", "float32")
        self.cfg, self.device = cfg, device
        self.f32 = dtype == "float32"
        self.elem = torch.float32 if self.f32 else BF16
        self.tp_rank, self.tp_size, self.tp_group = 0, 1, None
        self.use_coll, self.custom_ar, self.acts = False, None, None
        self.h = self.W = cfg.hidden_size
        self.V = cfg.vocab_size
        self.Vp = -(-self.V // 8) * 8                  # row stride of the bf16 logits (the sampling kernels read 16-byte chunks)
        self.block_size, self.max_blocks = block_size, max_blocks
        self.max_tokens = max_tokens
        self.max_logit_rows = max_logit_rows or max_tokens
        self.runs = cfg.runs()
        self.w: dict[str, torch.Tensor] = {}
        self.lam: list[float] = [0.0] * len(cfg.layers)
        self.kv: list[tuple[torch.Tensor, torch.Tensor]] = []
        self.tap_residuals: list | None = None         # tests: a list receives a copy of the residual rows after every layer run (eager only)

        def z(*shape, dtype=torch.float32):
            return torch.zeros(*shape, dtype=dtype, device=device)

        T, W, el = max_tokens, self.W, self.elem
        mix = [l.mixer for l in cfg.layers]
        mlps = [l.mlp for l in cfg.layers if l.mlp is not None]
        self.x = z(T, W)
        self.x0 = z(T, W) if cfg.loop_times > 1 and cfg.loop_stop > cfg.loop_start else None
        self.hn = z(T, W, dtype=el)
        self.y = z(T, W)
        self.qkvg = z(T * max(self._nqkvg(m) for m in mix))
        self.q = z(T * max(m.heads * 2 * m.dim for m in mix), dtype=el)
        self.gate = z(T * max(m.heads for m in mix))
        self.att = z(T * max(m.heads * m.vdim for m in mix), dtype=el)
        self.att_ws = z(256 * 4160)           # key-slice partials of the decode attention (csrc/attention_diff.hip): <= 256 slices in flight
        if mlps:
            top = max(m.top for m in mlps)
            self.r_idx = z(T * top, dtype=torch.int32)
            self.r_wt = z(T * top)
            self.r_z = z(T * max(m.experts for m in mlps))
            self.r_off = z(max(m.experts for m in mlps) + 1, dtype=torch.int32)
            self.r_perm = z(T * top, dtype=torch.int32)
            self.r_inv = z(T * top, dtype=torch.int32)
            self.act = z(T * max(m.top * m.ff for m in mlps), dtype=el)
            self.ydn = z(T * top * W)
            sff = max(m.shared_ff for m in mlps)
            self.sact = z(T * sff, dtype=el) if sff else None
            self.ysh = z(T, W) if sff else None
        R = self.max_logit_rows
        self.lastn = z(R, W, dtype=el)
        self.logits32 = z(R, self.V)
        self.logits = z(R, self.Vp, dtype=BF16)

    @staticmethod
    def _nqkvg(m) -> int:
        return m.heads * 2 * m.dim + m.kv_heads * 2 * m.dim + m.kv_heads * m.vdim + m.heads

    # ---------------------------------------------------------------------------------------------
    def load_weights(self, weight_iter) -> None:
        """Consumes (name, bf16 tensor) pairs under the checkpoint's names.  Per layer the q, k, v and gate matrices are stacked into one
        [q | k | v | g] projection, the experts' matrices into [E][ff][W] / [E][W][ff]; lambda is folded to one fp32 number."""
        raw = {n: t.to(self.device) for n, t in weight_iter}
        cv = lambda t: t.to(self.elem).contiguous()
        w = self.w = {}
        for n in ("embed", "final.norm", "head"):
            w[n] = cv(raw[n])
        for i, lc in enumerate(self.cfg.layers):
            p = f"l{i}."
            for n in ("norm1", "norm1b", "mix.q.norm", "mix.k.norm", "mix.o"):
                w[p + n] = cv(raw[p + n])
            w[p + "mix.qkvg"] = cv(torch.cat([raw[p + "mix.q"], raw[p + "mix.k"], raw[p + "mix.v"], raw[p + "mix.g"]], dim=0))
            f = lambda n: raw[p + "mix." + n].float()
            self.lam[i] = float(torch.exp((f("lq1") * f("lk1")).sum()) - torch.exp((f("lq2") * f("lk2")).sum()) + lc.mixer.diff)
            if lc.mlp is not None:
                for n in ("norm2", "norm2b", "mlp.router"):
                    w[p + n] = cv(raw[p + n])
                w[p + "mlp.up"] = cv(torch.stack([raw[p + f"mlp.e{e}.up"] for e in range(lc.mlp.experts)]))
                w[p + "mlp.down"] = cv(torch.stack([raw[p + f"mlp.e{e}.down"] for e in range(lc.mlp.experts)]))
                if lc.mlp.shared_ff:
                    w[p + "mlp.shared.up"] = cv(raw[p + "mlp.shared.up"])
                    w[p + "mlp.shared.down"] = cv(raw[p + "mlp.shared.down"])
        torch.cuda.synchronize(self.device)

    def weight_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for n, t in self.w.items() if n != "embed")

    def active_weight_bytes(self, T: int = 1) -> int:
        """HBM bytes of weights one forward of T tokens must stream at least: every dense matrix once per layer RUN, and of the experts
        min(E, T * top) per layer run."""
        per = {}
        for n, t in self.w.items():
            per[n] = t.numel() * t.element_size()
        total = per["head"] + per["final.norm"]
        for li, _ in self.runs:
            p, lc = f"l{li}.", self.cfg.layers[li]
            total += sum(per[p + n] for n in ("norm1", "norm1b", "mix.qkvg", "mix.o", "mix.q.norm", "mix.k.norm"))
            if lc.mlp is not None:
                frac = min(lc.mlp.experts, T * lc.mlp.top) / lc.mlp.experts
                total += int((per[p + "mlp.up"] + per[p + "mlp.down"]) * frac) + per[p + "mlp.router"] + per[p + "norm2"] + per[p + "norm2b"]
                if lc.mlp.shared_ff:
                    total += per[p + "mlp.shared.up"] + per[p + "mlp.shared.down"]
        return total

    def kv_block_bytes(self) -> int:
        es = 4 if self.f32 else 2
        return sum(self.cfg.layers[li].mixer.kv_heads * self.block_size * (2 * self.cfg.layers[li].mixer.dim + self.cfg.layers[li].mixer.vdim) * es
                   for li, _ in self.runs)

    def alloc_kv(self, num_blocks: int) -> None:
        """Per layer run: K [blocks][G][block_size][2 * dim] (both maps, normalised), V transposed per page [blocks][G][vdim][block_size]."""
        self.num_blocks = num_blocks
        self.kv = []
        for li, _ in self.runs:
            m = self.cfg.layers[li].mixer
            self.kv.append((torch.zeros(num_blocks, m.kv_heads, self.block_size, 2 * m.dim, dtype=self.elem, device=self.device),
                            torch.zeros(num_blocks, m.kv_heads, m.vdim, self.block_size, dtype=self.elem, device=self.device)))

    # ---------------------------------------------------------------------------------------------
    def launch_mixer(self, run: int, li: int, T: int, positions, meta: AttnMeta) -> None:
        """hn (normalised rows) -> y (fp32 mixer output rows)."""
        cfg, w, f = self.cfg, self.w, self.f32
        m, p = cfg.layers[li].mixer, f"l{li}.mix."
        kc, vc = self.kv[run]
        H.gemm_rows(self.hn, w[p + "qkvg"], self.qkvg, T, self._nqkvg(m), self.W, f)
        H.diffattn_store(self.qkvg, w[p + "q.norm"], w[p + "k.norm"], cfg.rms_norm_eps, meta.slot_mapping, self.q, self.gate, kc, vc,
                         T, m.heads, m.kv_heads, m.dim, m.vdim, self.block_size, f)
        H.diffattn_paged(self.q, kc, vc, self.gate, meta.block_tables, self.max_blocks, positions, meta.B, T, m.heads, m.kv_heads,
                         m.dim, m.vdim, self.block_size, m.scale, self.lam[li], 1.0 - m.diff, cfg.rms_norm_eps, self.att, f,
                         cu_q=meta.cu_q, q_per_seq=meta.q_per_seq, context_lens=meta.context_lens, max_q=meta.max_q,
                         workspace=self.att_ws, ctx_hint=meta.ctx_hint)
        H.gemm_rows(self.att, w[p + "o"], self.y, T, self.W, m.heads * m.vdim, f)

    def launch_mlp(self, li: int, T: int, combine: bool = True) -> None:
        """hn (normalised rows) -> y (fp32 feed-forward output rows); combine=False leaves the experts' rows in ydn / ysh for the
        fused tail (ssd_sandwich_tail)."""
        w, f, W = self.w, self.f32, self.W
        ml, p = self.cfg.layers[li].mlp, f"l{li}.mlp."
        H.gemm_rows(self.hn, w[p + "router"], self.r_z, T, ml.experts, W, f)
        H.moe_route(self.r_z, self.r_idx, self.r_wt, T, ml.experts, ml.top)
        H.moe_plan(self.r_idx, T, ml.top, ml.experts, self.r_off, self.r_perm, self.r_inv)
        H.gemm_rows_grouped(self.hn, w[p + "up"], self.act, self.r_off, ml.experts, T * ml.top, ml.ff, W, f, H.GR_RELU2,
                            row_idx=self.r_perm, idx_div=ml.top)
        H.gemm_rows_grouped(self.act, w[p + "down"], self.ydn, self.r_off, ml.experts, T * ml.top, W, ml.ff, f, H.GR_F32)
        if ml.shared_ff:
            H.gemm_rows(self.hn, w[p + "shared.up"], self.sact, T, ml.shared_ff, W, f, H.GR_RELU2)
            H.gemm_rows(self.sact, w[p + "shared.down"], self.ysh, T, W, ml.shared_ff, f)
        if combine:
            H.moe_combine(self.ydn, self.r_inv, self.r_wt, self.ysh if ml.shared_ff else None, self.y, T, ml.top, W)

    def forward(self, input_ids: torch.Tensor, positions: torch.Tensor, T: int, meta: AttnMeta) -> None:
        """Runs every layer run over the T token rows; leaves the fp32 residual rows in self.x."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        assert T <= self.max_tokens and meta.mode == H.MODE_CAUSAL and (meta.cu_q is not None or meta.q_per_seq > 0)
        eps = cfg.rms_norm_eps
        H.embed_res32(input_ids, w["embed"], self.x, self.x0, T, W, f)
        if self.tap_residuals is not None:
            return self._forward_unfused(positions, T, meta)
        # fused tails: every sublayer's post-norm + residual sum also writes the NEXT sublayer's normalised input (one launch; the
        # routed mix rides along), so only the first layer run has a norm launch of its own
        H.rmsnorm_res32(self.x, w[f"l{self.runs[0][0]}.norm1"], eps, self.hn, T, W, f)
        for run, (li, ps) in enumerate(self.runs):
            p, ml = f"l{li}.", cfg.layers[li].mlp
            nxt = {}
            if run + 1 < len(self.runs):
                nli, nps = self.runs[run + 1]
                nxt = dict(next_weight=w[f"l{nli}.norm1"], next_out=self.hn,
                           next_add=self.x0 if (nps > 0 and nli == cfg.loop_start) else None)     # the embedding output re-enters
            self.launch_mixer(run, li, T, positions, meta)
            if ml is None:
                H.sandwich_tail(w[p + "norm1b"], eps, self.x, T, W, f, y=self.y, **nxt)
                continue
            H.sandwich_tail(w[p + "norm1b"], eps, self.x, T, W, f, y=self.y, next_weight=w[p + "norm2"], next_out=self.hn)
            self.launch_mlp(li, T, combine=False)
            H.sandwich_tail(w[p + "norm2b"], eps, self.x, T, W, f, ydn=self.ydn, inv=self.r_inv, weights=self.r_wt,
                            shared=self.ysh if ml.shared_ff else None, top=ml.top, y_scratch=self.y, **nxt)

    def _forward_unfused(self, positions, T: int, meta: AttnMeta) -> None:
        """The same forward with one launch per step (norm, mix, post-norm + sum) and a copy of the residual rows after every layer
        run, before whatever precedes the next run (tests)."""
        cfg, w, f, W = self.cfg, self.w, self.f32, self.W
        eps = cfg.rms_norm_eps
        for run, (li, ps) in enumerate(self.runs):
            p = f"l{li}."
            again = self.x0 if (ps > 0 and li == cfg.loop_start) else None
            H.rmsnorm_res32(self.x, w[p + "norm1"], eps, self.hn, T, W, f, add=again)
            self.launch_mixer(run, li, T, positions, meta)
            H.rmsnorm_add_res32(self.y, w[p + "norm1b"], eps, self.x, T, W, f)
            if cfg.layers[li].mlp is not None:
                H.rmsnorm_res32(self.x, w[p + "norm2"], eps, self.hn, T, W, f)
                self.launch_mlp(li, T)
                H.rmsnorm_add_res32(self.y, w[p + "norm2b"], eps, self.x, T, W, f)
            self.tap_residuals.append(self.x[:T].clone())

    def compute_logits(self, T: int, gather: torch.Tensor | None = None, rows: int | None = None) -> int:
        """Final norm (optionally of the `gather` rows only) and the LM head: fp32 logits in logits32[:n], their bf16 rounding (row
        stride Vp, padding -inf) in logits[:n] for the sampling kernels.  Returns n."""
        n = T if gather is None else rows
        assert n <= self.max_logit_rows
        H.rmsnorm_res32(self.x, self.w["final.norm"], self.cfg.rms_norm_eps, self.lastn, n, self.W, self.f32, gather=gather)
        H.gemm_rows(self.lastn, self.w["head"], self.logits32, n, self.V, self.W, self.f32)
        H.rows_f32_to_bf16(self.logits32, self.logits, n, self.V, self.V, self.Vp)
        return n
