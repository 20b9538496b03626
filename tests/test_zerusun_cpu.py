"""CPU-side checks of the Zerusun integration: the config reader and its layer-run order, checkpoint names, state slots in the block
manager / scheduler / trace engine (a recording runner, no GPU), and the oracle's own mechanisms against hand-made cases and against
the restatements the kernels rest on (attention in the latent space, the recurrence as an explicit sum)."""
import json
import math

import pytest
import torch

from oracle import zerusun as Z
from ssd_amd.model_config import RopeSpec, ZerusunConfig, read_native_config
from ssd_amd.weights import param_shapes, synthetic_state_dict


def small_config(loop=(1, 3, 2)):
    return Z.make_config([Z.latent_layer(mlp=Z.dense_mlp()), Z.lightning_layer(mlp=Z.moe_mlp()), Z.lightning_layer(),
                          Z.latent_layer(window=0, scaling=None, mlp=Z.moe_mlp(groups=None, shared_ff=0))], loop=loop)


def test_config_reader_and_run_order(tmp_path):
    cfg = small_config()
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    c = read_native_config(str(tmp_path))
    assert isinstance(c, ZerusunConfig) and c.family == "zerusun" and c.recurrent and c.has_loop
    assert c.runs() == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (3, 0)] == [(i, t) for i, t, _ in Z.layer_runs(cfg)]
    assert [f for _, _, f in Z.layer_runs(cfg)] == [False, True, False, True, False, False]
    m0, m3 = c.layers[0].mixer, c.layers[3].mixer
    assert (m0.kind, m0.window, m0.rope.dims, m0.rope.scaling["factor"]) == ("latent_attention", 9, 8, 4.0)
    assert m3.window == 0 and m3.rope.scaling is None and c.layers[2].mlp is None
    r1, r3 = c.layers[1].mlp, c.layers[3].mlp
    assert (r1.groups, r1.keep, r1.scale, r1.shared_ff) == (2, 1, 1.5, 40) and (r3.groups, r3.keep, r3.shared_ff) == (1, 1, 0)
    assert c.layers[1].mixer.decay == cfg["layers"][1]["mixer"]["decay"]
    none = ZerusunConfig.from_json(small_config(loop=(2, 2, 3)))
    assert not none.has_loop and none.runs() == [(i, 0) for i in range(4)]
    whole = ZerusunConfig.from_json(small_config(loop=(0, 4, 2)))
    assert whole.runs() == [(i, t) for t in range(2) for i in range(4)]
    attn_only = ZerusunConfig.from_json(Z.make_config([Z.latent_layer()]))
    assert not attn_only.recurrent
    for breakit in (lambda d: d["layers"][0].update(type="conv"), lambda d: d["layers"][1]["mlp"].update(kind="glu"),
                    lambda d: d["layers"][1]["mixer"].update(decay=[0.5]), lambda d: d["layers"][1]["mlp"]["router"].update(top=5),
                    lambda d: d["layers"][0]["mixer"]["rot"].update(dims=10)):
        bad = small_config()
        breakit(bad)
        with pytest.raises(ValueError):
            ZerusunConfig.from_json(bad)


def test_checkpoint_names_cover_the_oracle_weights_and_synthetic_weights_load():
    for cfg in (small_config(), small_config(loop=(0, 0, 1))):
        c = ZerusunConfig.from_json(cfg)
        w = Z.random_model(cfg)
        assert {n: tuple(s) for n, s in param_shapes(c)} == {n: tuple(t.shape) for n, t in w.items()}
        sd = synthetic_state_dict(c, 0, 0.02)
        assert set(sd) == set(w) and all(sd[n].shape == w[n].shape for n in w)
        assert float(sd["final.norm.alpha"]) == 0.5 and float(sd["final.norm.b"].abs().max()) == 0.0


def test_rope_frequencies_of_the_reader_equal_the_oracle():
    for dims, base, sc in ((8, 10000.0, None), (32, 1e6, {"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0}),
                           (16, 500.0, {"factor": 8.0, "original": 64, "fast": 4.0, "slow": 0.5})):
        f, mag = RopeSpec(dims, base, sc).frequencies()
        fo, mo = Z.rope_frequencies(dims, base, sc)
        assert torch.allclose(torch.tensor(f, dtype=torch.float64), fo, rtol=1e-14, atol=0) and abs(mag - mo) < 1e-15
    f, mag = RopeSpec(8, 10000.0, None).frequencies()
    assert mag == 1.0 and f == [10000.0 ** (-2 * i / 8) for i in range(4)]
    # YaRN: the fastest pair keeps its frequency, the slowest is divided by the factor, everything lies between
    f, mag = RopeSpec(32, 1e6, {"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0}).frequencies()
    plain = [1e6 ** (-2 * i / 32) for i in range(16)]
    assert f[0] == plain[0] and abs(f[-1] - plain[-1] / 4.0) < 1e-18 and all(p / 4.0 - 1e-18 <= x <= p for x, p in zip(f, plain))
    assert abs(mag - (0.1 * math.log(4.0) + 1.0)) < 1e-15


def test_oracle_mechanisms_on_hand_made_cases():
    x = torch.tensor([[0.0, 1.0, -2.0]], dtype=torch.float64)
    assert torch.allclose(Z.dyt(x, torch.tensor([1.0, 2.0, 3.0]), torch.tensor([0.5, 0.0, -1.0]), 0.5),
                          torch.tensor([[0.5, 2 * math.tanh(0.5), 3 * math.tanh(-1.0) - 1.0]], dtype=torch.float64))
    assert torch.allclose(Z.rms(torch.tensor([[3.0, 4.0]], dtype=torch.float64), torch.ones(2), 0.0),
                          torch.tensor([[3.0, 4.0]], dtype=torch.float64) / math.sqrt(12.5))
    assert abs(float(Z.gelu_tanh(torch.tensor(1.0, dtype=torch.float64))) - 0.8411919906082768) < 1e-12
    # rotation: a quarter turn of the pair (i, i + dims / 2); entries past dims pass
    v = torch.tensor([[1.0, 2.0, 3.0, 4.0, 5.0]], dtype=torch.float64)
    out = Z.rope(v, torch.tensor([1]), torch.tensor([math.pi / 2, math.pi], dtype=torch.float64), 2.0, 4)
    assert torch.allclose(out, torch.tensor([[-6.0, -4.0, 2.0, -8.0, 5.0]], dtype=torch.float64), atol=1e-12)
    # router: 6 experts in 3 groups, the best 2 groups stay; expert 1 has the second largest score but its group loses to groups 1 and 2
    z = torch.log(torch.tensor([[0.10, 0.22, 0.05, 0.25, 0.15, 0.23]], dtype=torch.float64))
    idx, wt = Z.route(z, {"top": 3, "scale": 2.0, "groups": {"count": 3, "keep": 2}})
    assert idx.tolist() == [[3, 5, 4]]
    assert torch.allclose(wt, torch.tensor([[0.25, 0.23, 0.15]], dtype=torch.float64) / 0.63 * 2.0)
    idx, wt = Z.route(z, {"top": 2, "scale": 1.0, "groups": None})
    assert idx.tolist() == [[3, 5]] and abs(float(wt.sum()) - 1.0) < 1e-12


def test_oracle_recurrence_is_the_decayed_sum_and_attention_runs_in_the_latent_space():
    cfg = small_config()
    w = Z.random_model(cfg, 3)
    P = {n: t.double() for n, t in w.items()}
    T, W = 21, cfg["width"]
    h = torch.randn(T, W, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    # o_t = sum_{j <= t} decay^(t - j) (q_t . k_j) v_j
    m = cfg["layers"][1]["mixer"]
    Hh, D, Dv = m["heads"], m["dim"], m["vdim"]
    q, k, v = (Z.silu(h @ P["l1.mix." + n].T).view(T, Hh, d) for n, d in (("q", D), ("k", D), ("v", Dv)))
    dec = torch.tensor(m["decay"], dtype=torch.float64)
    age = (torch.arange(T)[:, None] - torch.arange(T)[None, :]).clamp(min=0)
    wgt = torch.einsum("ihd,jhd->hij", q, k) * (dec[:, None, None] ** age[None]) * (torch.arange(T)[:, None] >= torch.arange(T)[None, :])
    o = torch.einsum("hij,jhe->ihe", wgt, v).reshape(T, Hh * Dv)
    ref = (Z.rms(o, P["l1.mix.norm"], 1e-5) * torch.sigmoid(h @ P["l1.mix.g"].T)) @ P["l1.mix.o"].T
    assert torch.allclose(Z.lightning(h, P, "l1.mix.", m, 1e-5), ref, rtol=1e-9, atol=1e-9)
    # latent space: score = <W_uk^T q_unrot, c> + <q_rot, k_rot>, output = W_uv (sum_j p_j c_j): what the cache (c and k_rot only) allows
    m = cfg["layers"][0]["mixer"]
    Hh, D, R, Dv, Cr, win = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["mask"]["size"]
    pos = torch.arange(T)
    fr, mag = Z.rope_frequencies(m["rot"]["dims"], m["rot"]["base"], m["rot"]["scaling"])
    qq = (Z.rms(h @ P["l0.mix.dq"].T, P["l0.mix.dq.norm"], 1e-5) @ P["l0.mix.uq"].T).view(T, Hh, D + R)
    dkv = h @ P["l0.mix.dkv"].T
    c, kr = Z.rms(dkv[:, :Cr], P["l0.mix.dkv.norm"], 1e-5), Z.rope(dkv[:, Cr:], pos, fr, mag, m["rot"]["dims"])
    q_lat = torch.einsum("thd,hdc->thc", qq[..., :D], P["l0.mix.uk"].view(Hh, D, Cr))
    s = (torch.einsum("ihc,jc->hij", q_lat, c) + torch.einsum("ihr,jr->hij", Z.rope(qq[..., D:], pos, fr, mag, m["rot"]["dims"]), kr)) * m["scale"]
    d = pos[:, None] - pos[None, :]
    s = s.masked_fill(~((d >= 0) & (d < win))[None], float("-inf"))
    o_lat = torch.einsum("hij,jc->ihc", torch.softmax(s, -1), c) * torch.sigmoid(h @ P["l0.mix.g"].T)[..., None]
    out = torch.einsum("ihc,hvc->ihv", o_lat, P["l0.mix.uv"].view(Hh, Dv, Cr)).reshape(T, Hh * Dv) @ P["l0.mix.o"].T
    assert torch.allclose(Z.latent_attention(h, P, "l0.mix.", m, 1e-5), out, rtol=1e-9, atol=1e-9)


def test_state_slots_are_taken_and_returned_with_the_pages():
    from ssd_amd.engine.block_manager import BlockManager
    from ssd_amd.engine.sequence import Sequence
    Sequence.block_size = 16
    with pytest.raises(AssertionError):
        BlockManager(8, 16, state_slots=2)                    # a state cannot be rebuilt from cached pages
    bm = BlockManager(8, 16, prefix_cache=False, state_slots=2)
    a, b, c = Sequence([1] * 20), Sequence([2] * 5), Sequence([3] * 5)
    bm.allocate(a)
    bm.allocate(b)
    assert (a.state_slot, b.state_slot) == (0, 1) and not bm.can_allocate(c)          # pages are free, slots are not
    bm.deallocate(a)
    assert a.state_slot == -1 and bm.can_allocate(c)
    bm.allocate(c)
    assert c.state_slot == 0
    bm.deallocate(c)
    bm.deallocate(b)
    assert bm.free_state_slots == [0, 1] and len(bm.free_block_ids) == 8
    plain = BlockManager(8, 16)
    plain.allocate(a)
    assert a.state_slot == -1


class _Recorder:
    """Stands in for the ModelRunner: records what every step would run."""

    def __init__(self, config):
        self.calls = []

    def run_rows(self, seqs, want):
        self.calls.append([(s.state_slot, list(s.block_table), s.num_cached_tokens, len(s)) for s in seqs])
        return torch.zeros(sum(len(w) for w in want), 4)


def test_scheduler_and_trace_engine_hand_out_state_slots(tmp_path):
    from ssd_amd.config import Config
    from ssd_amd.engine.scheduler import Scheduler
    from ssd_amd.engine.sequence import Sequence
    from ssd_amd.engine.trace_engine import TraceEngine
    (tmp_path / "config.json").write_text(json.dumps(small_config()))
    eng = TraceEngine(str(tmp_path), max_tokens=128, block_size=16, max_live=2, runner_factory=_Recorder)
    eng.step([{"id": "a", "tokens": [1] * 10, "want": [9]}, {"id": "b", "tokens": [2] * 3, "want": []}])
    assert [c[0] for c in eng.runner.calls[-1]] == [0, 1]
    with pytest.raises(RuntimeError):
        eng.step([{"id": "c", "tokens": [3], "want": []}])
    eng.step([{"id": "b", "tokens": [2], "want": []}], end=["a"])
    eng.step([{"id": "c", "tokens": [3] * 4, "want": []}])
    assert eng.runner.calls[-1][0][0] == 0 and eng.live["b"].state_slot == 1               # a's slot is in use again
    eng.step([], end=["b", "c"])
    assert eng.blocks.free_state_slots == [0, 1]
    # the scheduler: admission stops when the slots are out, a finished or preempted sequence gives its slot back, no prefix reuse
    cfg = Config(str(tmp_path), max_num_seqs=2, kvcache_block_size=16, num_kvcache_blocks=16, max_model_len=128, max_num_batched_tokens=128)
    Sequence.block_size = 16
    sch = Scheduler(cfg)
    assert not sch.block_manager.prefix_cache
    seqs = [Sequence([5] * 16) for _ in range(3)]
    for s in seqs:
        sch.add(s)
    picked, prefill = sch.schedule()
    assert prefill and picked == seqs[:2] and [s.state_slot for s in seqs] == [0, 1, -1]
    sch.postprocess(picked, [7, 7], True)
    sch.preempt(sch.running.pop())
    assert seqs[1].state_slot == -1 and seqs[1].num_cached_tokens == 0
    picked, prefill = sch.schedule()
    assert prefill and picked == [seqs[1]] and seqs[1].state_slot == 1
    with pytest.raises(AssertionError):
        Config(str(tmp_path), speculate=True, draft=str(tmp_path), speculate_k=2, kvcache_block_size=16)


def test_bench_option_and_equal_size_pairs():
    """bench.py accepts --workload zerusun next to its default; every benchmarked size pairs a Zerusun model with a Fatulix model of the
    same width, layers, vocabulary, experts, top and feed-forward parameters per token."""
    import bench
    from ssd_amd.utils import arch_bench
    assert bench.parse([]).workload == "c4"                                  # the default workload is untouched
    a = bench.parse(["--workload", "zerusun", "--arch-size", "w2048", "--arch-batch", "1", "--arch-only", "zerusun"])
    assert a.workload == "zerusun" and a.arch_size == "w2048" and a.arch_batch == 1 and a.arch_only == "zerusun"
    for size in arch_bench.SIZES:
        zer, fat = arch_bench.zerusun_models(size)
        assert zer.hidden_size == fat.hidden_size and zer.vocab_size == fat.vocab_size and len(zer.runs()) == len(fat.runs())
        assert {l.mixer.kind for l in zer.layers} == {"latent_attention", "lightning"} and zer.recurrent
        mz, mf = zer.layers[0].mlp, fat.layers[0].mlp
        assert (mz.experts, mz.top) == (mf.experts, mf.top)
        assert 3 * (mz.top * mz.ff + mz.shared_ff) == 2 * (mf.top * mf.ff + mf.shared_ff)
