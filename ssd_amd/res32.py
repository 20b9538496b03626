"""What the decoders with an fp32 residual stream and their own config.json share towards the ModelRunner: the LM-head outputs (fp32
logits + their bf16 rounding for the sampling kernels), greedy argmax, and weight replacement.  A subclass provides load_weights,
alloc_kv, kv_block_bytes, forward and compute_logits, and allocates logits32 [rows][V] (fp32) and logits [rows][Vp] (bf16)."""
from __future__ import annotations

import torch

from ssd_amd.hip import ops as H


class Res32Decoder:
    supports_float32 = True
    state_slots = 0                 # recurrent-state slots the model holds (0: every layer's memory is cache pages)

    def overwrite_weights(self, weight_iter) -> None:
        old, self.w = self.w, {}
        self.load_weights(weight_iter)
        new, self.w = self.w, old
        for n, t in new.items():
            old[n].copy_(t)
        torch.cuda.synchronize(self.device)

    def has_argmax_parts(self, n: int) -> bool:
        return False

    def argmax(self, n: int, out: torch.Tensor, out2: torch.Tensor | None = None, out3=None, out3_stride: int = 0) -> None:
        assert out3 is None
        H.argmax_rows(self.logits, self.Vp, n, self.V, out, out2)

    def full_logits(self, n: int) -> torch.Tensor:
        return self.logits[:n] if self.Vp == self.V else self.logits[:n, :self.V].contiguous()

    def logits_f32(self, n: int) -> torch.Tensor:
        return self.logits32[:n]
