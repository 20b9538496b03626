"""CPU-side checks of the Fatulix integration: the config reader and its layer-run order, checkpoint names, the oracle's own
mechanisms against hand-made cases, and the trace engine's page accounting with a recording runner (no GPU)."""
import json
import math

import pytest
import torch

from oracle import fatulix as F
from ssd_amd.model_config import FatulixConfig, read_native_config
from ssd_amd.weights import param_shapes, synthetic_state_dict


def test_config_reader_and_run_order(tmp_path):
    cfg = F.make_config(n_layers=5, loop=(1, 3, 3), no_mlp_layers=(4,), shared_ff=0)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    c = read_native_config(str(tmp_path))
    assert isinstance(c, FatulixConfig) and c.family == "fatulix"
    assert c.runs() == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (1, 2), (2, 2), (3, 0), (4, 0)] == F.layer_runs(cfg)
    assert c.num_layers == 9 and c.layers[4].mlp is None and c.layers[0].mlp.shared_ff == 0
    assert FatulixConfig.from_json(F.make_config(n_layers=2, loop=(0, 0, 1))).runs() == [(0, 0), (1, 0)]
    assert FatulixConfig.from_json(F.make_config(n_layers=2, loop=(0, 2, 2))).runs() == [(0, 0), (1, 0), (0, 1), (1, 1)]
    (tmp_path / "config.json").write_text(json.dumps({"model_type": "llama"}))
    assert read_native_config(str(tmp_path)) is None          # other directories go through the transformers reader
    bad = F.make_config(n_layers=1)
    bad["layers"][0]["type"] = "recurrent"
    with pytest.raises(ValueError):
        FatulixConfig.from_json(bad)


def test_checkpoint_names_cover_the_oracle_weights_and_synthetic_weights_load():
    cfg = F.make_config(n_layers=3, no_mlp_layers=(1,), experts=3)
    c = FatulixConfig.from_json(cfg)
    w = F.random_model(cfg)
    assert {n: tuple(s) for n, s in param_shapes(c)} == {n: tuple(t.shape) for n, t in w.items()}
    sd = synthetic_state_dict(c, 0, 0.02)
    assert set(sd) == set(w) and all(sd[n].shape == w[n].shape for n in w)


def test_oracle_mechanisms_on_hand_made_cases():
    x = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    assert torch.allclose(F.rms(x, 0.0), x / math.sqrt(12.5))
    # softmax over the chosen logits only, largest first
    idx, wt = F.route(torch.eye(3, dtype=torch.float64), torch.tensor([[1.0, 0, 0], [3.0, 0, 0], [2.0, 0, 0], [0, 5.0, 0]], dtype=torch.float64), 2)
    assert idx[0].tolist() == [1, 2] and torch.allclose(wt[0], torch.softmax(torch.tensor([3.0, 2.0], dtype=torch.float64), 0))
    assert idx[1].tolist()[0] == 3
    # an expert is W_down relu(W_up h)^2
    assert torch.allclose(F.expert(torch.tensor([2.0, -1.0]), torch.tensor([[1.0, 0], [0, 1.0]]), torch.tensor([[1.0, 1.0]])), torch.tensor([4.0]))
    # causal: the first position sees itself only
    p = F.causal_softmax(torch.zeros(3, 3, dtype=torch.float64))
    assert torch.allclose(p, torch.tensor([[1, 0, 0], [.5, .5, 0], [1 / 3, 1 / 3, 1 / 3]], dtype=torch.float64))


def test_oracle_differential_attention_reduces_to_its_definition():
    """One head, keys made so that map 1 looks at position 0 and map 2 at the query's own position: o = rms(v_0 - lambda v_i)."""
    cfg = F.make_config(n_layers=1, heads=1, kv_heads=1, dim=4, vdim=6, width=8, diff=0.2, scale=50.0, experts=2, top=1)
    m = cfg["layers"][0]["mixer"]
    T, big = 5, 1.0
    g = torch.Generator().manual_seed(0)
    h = torch.randn(T, 8, generator=g, dtype=torch.float64)
    w = {k: v.double() for k, v in F.random_model(cfg).items()}
    out = F.diff_attention(h, w, "l0.mix.", m, 1e-5, torch.float64)
    # independent restatement with explicit loops over positions
    q = (h @ w["l0.mix.q"].T).view(T, 2, 4)
    k = (h @ w["l0.mix.k"].T).view(T, 2, 4)
    v = h @ w["l0.mix.v"].T
    q = F.rms(q, 1e-5) * w["l0.mix.q.norm"]
    k = F.rms(k, 1e-5) * w["l0.mix.k.norm"]
    lam = math.exp(float((w["l0.mix.lq1"] * w["l0.mix.lk1"]).sum())) - math.exp(float((w["l0.mix.lq2"] * w["l0.mix.lk2"]).sum())) + 0.2
    rows = []
    for i in range(T):
        a = []
        for mp in range(2):
            s = torch.stack([(q[i, mp] * k[j, mp]).sum() * 50.0 for j in range(i + 1)])
            a.append((torch.softmax(s, 0)[:, None] * v[:i + 1]).sum(0))
        o = a[0] - lam * a[1]
        o = o / torch.sqrt((o * o).mean() + 1e-5) * 0.8 * torch.sigmoid(h[i] @ w["l0.mix.g"][0])
        rows.append(o)
    ref = torch.stack(rows) @ w["l0.mix.o"].T
    assert torch.allclose(out, ref, atol=1e-10)


class _Recorder:
    """Stands in for the ModelRunner: records what each step would run."""

    def __init__(self, config):
        self.config, self.calls = config, []

    def run_rows(self, seqs, want):
        self.calls.append([(list(s.block_table), s.num_cached_tokens, len(s), list(w)) for s, w in zip(seqs, want)])
        return torch.zeros(sum(len(w) for w in want), 4)


def test_trace_engine_takes_and_returns_pages():
    from ssd_amd.engine.trace_engine import TraceEngine
    eng = TraceEngine("llama-3.2-1b", max_tokens=200, block_size=64, runner_factory=_Recorder)      # 4 pages (200 rounds up to 256)
    assert len(eng.blocks.free_block_ids) == 4
    out = eng.step([{"id": "a", "tokens": list(range(65)), "want": [0, 64]}, {"id": "b", "tokens": [1], "want": []}])
    assert out.shape[0] == 2 and len(eng.blocks.free_block_ids) == 1
    a0 = eng.runner.calls[-1][0]
    assert a0[1:] == (0, 65, [0, 64]) and len(a0[0]) == 2
    assert eng.step([{"id": "b", "tokens": [2, 3], "want": []}], end=["a"]) is None
    assert eng.runner.calls[-1][0][1:3] == (1, 3) and len(eng.blocks.free_block_ids) == 3
    eng.step([{"id": "c", "tokens": list(range(130)), "want": [129]}])           # reuses the pages a gave back
    assert set(eng.runner.calls[-1][0][0]) & set(a0[0])
    with pytest.raises(RuntimeError):
        eng.step([{"id": "d", "tokens": [5], "want": []}])                          # no page left
    eng.step([], end=["b", "c"])
    assert len(eng.blocks.free_block_ids) == 4 and not eng.live


def test_bench_option_and_equal_size_pairs():
    """bench.py accepts --workload fatulix next to its default; every benchmarked size pairs a Fatulix model with a Llama decoder of the
    same width, projection sizes and feed-forward parameters per token."""
    import bench
    from ssd_amd.utils import arch_bench
    assert bench.parse([]).workload == "c4"                                  # the default workload is untouched
    a = bench.parse(["--workload", "fatulix", "--arch-size", "w2048", "--arch-batch", "1"])
    assert a.workload == "fatulix" and a.arch_size == "w2048" and a.arch_batch == 1
    for size in arch_bench.SIZES:
        fat, llama = arch_bench.models(size)
        m, ml = fat.layers[0].mixer, fat.layers[0].mlp
        assert fat.hidden_size == llama.hidden_size and fat.vocab_size == llama.vocab_size and len(fat.layers) == llama.num_layers
        assert m.heads * 2 * m.dim == llama.q_size and m.kv_heads * 2 * m.dim == llama.kv_size == m.kv_heads * m.vdim
        assert ml.top * 2 * ml.ff + 2 * ml.shared_ff == 3 * llama.intermediate_size
