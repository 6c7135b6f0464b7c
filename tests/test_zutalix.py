"""Zutalix family on the CPU path (fp32) against the plain float64 oracle in
tests/hybrid_oracle.py: every mechanism alone, then whole models through the
engine's segment step, cache / slot reuse, and greedy generation through
generate() and the scheduler. Configurations are small and deliberately
lopsided: grouped heads everywhere, partial rotary width, value sizes that
differ from key sizes, unequal low-rank widths, layers of different shapes,
a delta layer first and with a feed-forward, a parallel layer without one."""

import json
import os

import pytest
import torch

import hybrid_oracle as O
from kllms_amd.engine.config import (BlockAttnSpec, ChannelDeltaSpec, DecayLinearAttnSpec, EngineConfig,
                                     GluSpec, ParallelMixerSpec, RotarySpec)
from kllms_amd.engine.engine import GenRequest, LLMEngine
from kllms_amd.engine.kvcache import HybridStateCache, LayerCacheSpec, SequenceKV
from kllms_amd.engine.sampling import SamplingParams
from kllms_amd.engine.scheduler import BatchScheduler
from kllms_amd.models.llama import ForwardBatch
from kllms_amd.models.mixers import ChannelDeltaMixer, ClampedGLU, ParallelMixer, rotary_inv_freq

EPS = 1e-5
SCALING = {"factor": 3.0, "high": 3.0, "low": 1.0, "original": 40}


def par(heads=4, kv=2, dim=12, mask=24, rdims=8, lh=3, ld=6, lv=10, ff=40, limit=0.7, scaling=SCALING, mlp=True):
    return {"type": "parallel",
            "mixer": {"left": {"dim": dim, "vdim": dim, "heads": heads, "kv_heads": kv, "scale": 0.4,
                               "mask": {"size": mask},
                               "rot": {"base": 100.0, "dims": rdims, "scaling": scaling}},
                      "right": {"dim": ld, "vdim": lv, "heads": lh,
                                "decay": [0.5, 0.9, 0.97, 0.995][:lh]}},
            "mlp": {"kind": "dense", "ff": ff, "limit": limit} if mlp else None}


def delta(heads=4, kv=2, dim=6, vdim=10, conv=3, mlp=None):
    return {"type": "channel_delta",
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp}


CFG_A = {"architecture": "Zutalix", "vocab": 61, "width": 24, "norm": {"eps": EPS},
         "layers": [par(), delta(), par(mask=16, heads=2, kv=1, dim=8, rdims=8, lh=2, ld=4, lv=4, scaling=None)]}
# delta first and with a feed-forward, parallel without one, 5 taps, 1 kv group
CFG_B = {"architecture": "Zutalix", "vocab": 47, "width": 20, "norm": {"eps": 1e-6},
         "layers": [delta(heads=3, kv=1, dim=4, vdim=6, conv=5, mlp={"kind": "dense", "ff": 28, "limit": 1.5}),
                    par(heads=3, kv=3, dim=6, mask=7, rdims=2, lh=1, ld=8, lv=6, mlp=False),
                    delta(heads=2, kv=2, dim=8, vdim=4, conv=2)]}


def write_model(tmp, cfg, seed=0):
    from safetensors.torch import save_file

    w = O.random_weights(cfg, seed)
    # unequal bottlenecks for the two low-rank projections
    for i, sp in enumerate(cfg["layers"]):
        if sp["type"] == "channel_delta":
            p = f"l{i}.mix."
            g = torch.Generator().manual_seed(100 + i)
            r = w[p + "g1"].shape[0] + 3
            w[p + "g1"] = (torch.randn(r, cfg["width"], generator=g) * 0.3).bfloat16().float()
            w[p + "g2"] = (torch.randn(w[p + "g2"].shape[0], r, generator=g) * 0.3).bfloat16().float()
    os.makedirs(tmp, exist_ok=True)
    save_file({k: v.bfloat16().contiguous() for k, v in w.items()}, os.path.join(tmp, "model.safetensors"))
    with open(os.path.join(tmp, "config.json"), "w") as f:
        json.dump(cfg, f)
    return w


def make_engine(path, blocks=64, slots=4, **kw):
    return LLMEngine(EngineConfig(model=str(path), dtype="float32", device="cpu", max_kv_blocks=blocks,
                                  max_state_slots=slots, use_hip_graphs=False, **kw))


@pytest.fixture(scope="module")
def model_a(tmp_path_factory):
    d = tmp_path_factory.mktemp("zut_a")
    w = write_model(str(d), CFG_A, seed=1)
    return CFG_A, w, make_engine(d)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    d = tmp_path_factory.mktemp("zut_b")
    w = write_model(str(d), CFG_B, seed=2)
    return CFG_B, w, make_engine(d, blocks=40, slots=3)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def check(got, want, atol=2e-4):
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=atol)


# --- mechanisms alone -----------------------------------------------------------

def seg_batch(cache, seqs, counts):
    """Segment batch continuing each sequence by counts[b] rows."""
    pos, tseg, cu, slots, starts = [], [], [0], [], []
    for b, (seq, n) in enumerate(zip(seqs, counts)):
        starts.append(seq.num_tokens)
        pos += list(range(seq.num_tokens, seq.num_tokens + n))
        slots += cache.extend(seq, n)
        tseg += [b] * n
        cu.append(cu[-1] + n)
    width = max(len(s.blocks) for s in seqs)
    bt = torch.zeros(len(seqs), width, dtype=torch.int32)
    for b, s in enumerate(seqs):
        bt[b, :len(s.blocks)] = torch.tensor(s.blocks, dtype=torch.int32)
    i32 = lambda x: torch.tensor(x, dtype=torch.int32)
    return ForwardBatch(mode="segments", positions=torch.tensor(pos), slot_mapping=torch.tensor(slots),
                        kv_caches=cache.layer_caches(), cu_seqlens=i32(cu), block_tables=bt,
                        seg_start=i32(starts), state_slots=i32([s.state_slot for s in seqs]), token_seg=i32(tseg))


def run_mixer(mod, spec, h, cuts):
    """Feed h [L, W] through a mixer in portions; returns per-row outputs."""
    cache = HybridStateCache([spec], 4, 200, 3, "cpu", torch.float32)
    cache.slots.alloc()                       # the sequence does not get slot 0
    seq = cache.open_sequence()
    outs, at = [], 0
    for n in cuts:
        batch = seg_batch(cache, [seq], [n])
        y = mod(h[at:at + n].float(), batch, cache.layer_caches()[0])
        outs.append(y if isinstance(y, tuple) else (y,))
        at += n
    return [torch.cat([o[i] for o in outs]) for i in range(len(outs[0]))]


def load_module(mod, w, pre):
    for name, dst in mod.checkpoint_map(pre).items():
        dst.copy_(w[name].to(dst.dtype))


def spiky_input(L, W, spikes, seed=0):
    """Random rows with a few rows scaled up: their keys dominate every
    softmax that can see them, so a mask that is one position off shows."""
    h = torch.randn(L, W, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)
    for p in spikes:
        if p < L:
            h[p] *= 6.0
    return h


def parallel_specs(layer):
    le, ri = layer["mixer"]["left"], layer["mixer"]["right"]
    return ParallelMixerSpec(
        left=BlockAttnSpec(heads=le["heads"], kv_heads=le["kv_heads"], dim=le["dim"], vdim=le["vdim"],
                           scale=le["scale"], mask_size=le["mask"]["size"],
                           rot=RotarySpec(base=le["rot"]["base"], dims=le["rot"]["dims"],
                                          scaling=le["rot"]["scaling"])),
        right=DecayLinearAttnSpec(heads=ri["heads"], dim=ri["dim"], vdim=ri["vdim"], decay=ri["decay"]))


def test_rotary_frequencies_all_bands():
    rot = {"base": 100.0, "dims": 16, "scaling": SCALING}
    want = O.rotary_freqs(rot)
    # the three regimes are all present: kept, blended, slowed
    plain = [100.0 ** (-2 * i / 16) for i in range(8)]
    ratios = [a / b for a, b in zip(want, plain)]
    assert any(abs(r - 1) < 1e-12 for r in ratios) and any(abs(r - 1 / 3) < 1e-12 for r in ratios)
    assert any(1 / 3 + 1e-6 < r < 1 - 1e-6 for r in ratios)
    got = rotary_inv_freq(RotarySpec(base=100.0, dims=16, scaling=SCALING))
    torch.testing.assert_close(got.double(), torch.tensor(want, dtype=torch.float64), rtol=1e-6, atol=0)


@pytest.mark.parametrize("cuts", [[75], [40] + [1] * 35, [2, 5, 16, 1, 2, 31, 3, 15], [23, 2, 24, 1, 25]])
def test_parallel_mixer_edges(cuts):
    """Block-local attention + decayed linear attention against the oracle,
    with dominant keys at block starts / ends, page borders and far back."""
    layer = par(mask=24)
    cfg = {"vocab": 8, "width": 24, "norm": {"eps": EPS}, "layers": [layer]}
    w = O.random_weights(cfg, 3)
    L = sum(cuts)
    # block edges (23|24, 47|48), page borders (4-token pages: 3|4, 15|16), first tokens, far back
    h = spiky_input(L, 24, [0, 1, 3, 4, 15, 16, 23, 24, 25, 47, 48, 49, 71, 72], seed=4)
    mod = ParallelMixer(parallel_specs(layer), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    mod.inp.bias[mod.inp.parts["right.q"][0]:].zero_()
    left, right = run_mixer(mod, LayerCacheSpec(kv=(2, 12, 12), rec=(3, 6, 10)), h, cuts)
    w64 = {k: v.double() for k, v in w.items()}
    check(left, O.chunk_softmax_attention(h, w64, "l0.mix.left.", layer["mixer"]["left"], EPS))
    check(right, O.decayed_linear_attention(h, w64, "l0.mix.right.", layer["mixer"]["right"], EPS))


def test_block_mask_is_visible_in_the_output():
    """The oracle comparison above only bites if a dominant key really changes
    the result across the block edge: position 24 (first of its block) must
    ignore the spike at 23, position 23 must see the one at 0."""
    layer = par(mask=24)
    cfg = {"vocab": 8, "width": 24, "norm": {"eps": EPS}, "layers": [layer]}
    w64 = {k: v.double() for k, v in O.random_weights(cfg, 3).items()}
    a = spiky_input(30, 24, [23], seed=4)
    b = a.clone()
    b[23] /= 6.0
    ya = O.chunk_softmax_attention(a, w64, "l0.mix.left.", layer["mixer"]["left"], EPS)
    yb = O.chunk_softmax_attention(b, w64, "l0.mix.left.", layer["mixer"]["left"], EPS)
    assert (ya[24:] - yb[24:]).abs().max() < 1e-12 and (ya[23] - yb[23]).abs().max() > 1e-2


@pytest.mark.parametrize("cuts", [[40], [30] + [1] * 10, [1, 2, 1, 3, 2, 31], [2] * 20])
@pytest.mark.parametrize("conv", [1, 2, 4, 6])
def test_channel_delta_mixer(cuts, conv):
    layer = delta(heads=4, kv=2, dim=6, vdim=10, conv=conv)
    cfg = {"vocab": 8, "width": 24, "norm": {"eps": EPS}, "layers": [layer]}
    w = O.random_weights(cfg, 5)
    h = spiky_input(sum(cuts), 24, [0, 2, 17], seed=6)
    m = layer["mixer"]
    r = w["l0.mix.a1"].shape[0]
    mod = ChannelDeltaMixer(ChannelDeltaSpec(heads=4, kv_heads=2, dim=6, vdim=10, conv=conv, decay_rank=r,
                                             gate_rank=r), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    (y,) = run_mixer(mod, mod.cache_spec(), h, cuts)
    check(y, O.channel_delta_mixer(h, {k: v.double() for k, v in w.items()}, "l0.mix.", m, EPS))


def test_clamped_glu_both_clamps_active():
    cfg = {"vocab": 8, "width": 24, "norm": {"eps": EPS}, "layers": [par(ff=40, limit=0.7)]}
    w = O.random_weights(cfg, 7)
    h = torch.randn(9, 24, dtype=torch.float64, generator=torch.Generator().manual_seed(8)) * 3
    mod = ClampedGLU(GluSpec(ff=40, limit=0.7), 24, torch.float32)
    load_module(mod, w, "l0.mlp.")
    w64 = {k: v.double() for k, v in w.items()}
    g, u = h @ w64["l0.mlp.gate"].T, h @ w64["l0.mlp.up"].T
    assert (g > 0.7).any() and (u > 0.7).any() and (u < -0.7).any() and (g < -0.7).any()
    check(mod(h.float()), O.clamped_glu(h, w64, "l0.mlp.", {"limit": 0.7}))


# --- whole models through the engine ---------------------------------------------

def run_schedule(eng, schedule, prompts):
    """schedule: list of steps, each [(request, n_tokens)]; every row's logits
    are collected. Requests are freed when they run out of tokens."""
    seqs, at, got = {}, {}, {r: [] for r in prompts}
    for step in schedule:
        entries, names = [], []
        for r, n in step:
            if r not in seqs:
                seqs[r], at[r] = eng.open_sequence(), 0
            entries.append((seqs[r], prompts[r][at[r]:at[r] + n], list(range(n))))
            names.append((r, n))
            at[r] += n
        lg = eng.step_segments(entries)
        o = 0
        for r, n in names:
            got[r].append(lg[o:o + n])
            o += n
            if at[r] == len(prompts[r]):
                eng.kv.free_sequence(seqs.pop(r))
    return {r: torch.cat(v) for r, v in got.items() if v}


def test_whole_prompt_and_first_tokens(model_a):
    cfg, w, eng = model_a
    p = toks(70, cfg["vocab"], 1)
    got = run_schedule(eng, [[("x", 70)]], {"x": p})["x"]
    want = O.forward(cfg, w, p)
    check(got, want)
    check(got[:3], want[:3], atol=5e-5)      # the first tokens of a sequence
    one = run_schedule(eng, [[("y", 1)]], {"y": p[:1]})["y"]
    check(one, want[:1])


def test_prefill_then_decode_long(model_a):
    """4 prompt tokens, then 150 single-token steps: several attention
    blocks, many pages, long recurrences."""
    cfg, w, eng = model_a
    p = toks(154, cfg["vocab"], 2)
    got = run_schedule(eng, [[("x", 4)]] + [[("x", 1)]] * 150, {"x": p})["x"]
    check(got, O.forward(cfg, w, p), atol=5e-4)


@pytest.mark.parametrize("cuts", [[2, 5, 16, 1, 2, 31, 3, 12], [2] * 15 + [1] * 6, [17, 15, 16, 1, 1, 22]])
def test_portions(model_a, cuts):
    cfg, w, eng = model_a
    p = toks(sum(cuts), cfg["vocab"], 3)
    got = run_schedule(eng, [[("x", n)] for n in cuts], {"x": p})["x"]
    check(got, O.forward(cfg, w, p))


def test_mixed_batches_reuse_blocks_and_slots(model_b):
    """Unequal requests side by side (portions beside single tokens), more
    requests than slots and more tokens than blocks over the run, so freed
    pages and slots change hands; each request must match itself alone."""
    cfg, w, eng = model_b
    L = {"a": 50, "b": 23, "c": 37, "d": 41, "e": 9, "f": 30}
    prompts = {r: toks(n, cfg["vocab"], 10 + i) for i, (r, n) in enumerate(L.items())}
    sched = [[("a", 16)], [("a", 3), ("b", 20)], [("a", 1), ("b", 1), ("c", 30)], [("a", 10), ("b", 2), ("c", 1)],
             [("a", 20), ("c", 6)],                                  # b and then a, c finish
             [("d", 2), ("e", 8)], [("d", 1), ("e", 1), ("f", 7)], [("d", 30), ("f", 1)], [("d", 8), ("f", 22)]]
    assert sum(L.values()) > eng.kv.num_blocks * eng.kv.block_size / 4
    got = run_schedule(eng, sched, prompts)
    for r in L:
        check(got[r], O.forward(cfg, w, prompts[r]))
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots
    assert eng.kv.allocator.num_free == eng.kv.num_blocks


def test_slot_state_is_not_inherited(model_b):
    """A slot and pages last used by a long request go to a new one: its
    first step must start from zero state."""
    cfg, w, eng = model_b
    a, b = toks(45, cfg["vocab"], 20), toks(6, cfg["vocab"], 21)
    run_schedule(eng, [[("a", 45)]], {"a": a})
    got = run_schedule(eng, [[("b", 2)], [("b", 1)], [("b", 3)]], {"b": b})["b"]
    check(got, O.forward(cfg, w, b))


def test_other_shapes(model_b):
    cfg, w, eng = model_b
    p = toks(33, cfg["vocab"], 30)
    got = run_schedule(eng, [[("x", 9)], [("x", 1)], [("x", 1)], [("x", 22)]], {"x": p})["x"]
    check(got, O.forward(cfg, w, p))


def oracle_greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(O.forward(cfg, w, ids)[-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_and_fork(model_a):
    cfg, w, eng = model_a
    # token ids the byte tokenizer's eos would stop on are avoided by vocab < 256
    p1, p2 = toks(21, cfg["vocab"], 40), toks(5, cfg["vocab"], 41)
    sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
    outs = eng.generate([GenRequest(prompt_ids=p1, n=2, sampling=sp(7)), GenRequest(prompt_ids=p2, n=1, sampling=sp(9))])
    want1, want2 = oracle_greedy(cfg, w, p1, 7), oracle_greedy(cfg, w, p2, 9)
    assert [s.token_ids for s in outs[0].streams] == [want1, want1]
    assert outs[1].streams[0].token_ids == want2
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots and eng.kv.allocator.num_free == eng.kv.num_blocks


def test_scheduler_chunked_prefill_and_merge(tmp_path):
    w = write_model(str(tmp_path), CFG_A, seed=1)
    eng = make_engine(tmp_path, blocks=128, slots=8, prefill_chunk_tokens=8, max_batch_size=4)
    sched = BatchScheduler(eng)
    try:
        p1, p2 = toks(29, CFG_A["vocab"], 50), toks(6, CFG_A["vocab"], 51)
        sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
        f1 = sched.submit(GenRequest(prompt_ids=p1, n=1, sampling=sp(6)))     # prefilled in slices of 8
        f2 = sched.submit(GenRequest(prompt_ids=p2, n=2, sampling=sp(8)))
        o1, o2 = f1.result(timeout=120), f2.result(timeout=120)
    finally:
        sched.shutdown()
    assert o1.streams[0].token_ids == oracle_greedy(CFG_A, w, p1, 6)
    want2 = oracle_greedy(CFG_A, w, p2, 8)
    assert [s.token_ids for s in o2.streams] == [want2, want2]
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots


def test_config_reader_takes_sizes_from_file_and_tensors(tmp_path):
    write_model(str(tmp_path), CFG_B, seed=2)
    arch = EngineConfig(model=str(tmp_path)).resolve_arch()
    assert arch.arch == "zutalix" and arch.vocab_size == 47 and arch.hidden_size == 20
    d0 = arch.layers[0].channel_delta
    assert (d0.conv, d0.kv_heads, d0.gate_rank - d0.decay_rank) == (5, 1, 3)
    assert arch.layers[0].mlp.ff == 28 and arch.layers[1].mlp is None
    assert arch.layers[1].parallel.left.rot.dims == 2 and arch.layers[1].parallel.left.mask_size == 7


def test_trace_replay_cli(tmp_path, model_b):
    """bin/trace_run end to end on a tiny model: files, 'done' lines, reuse."""
    import subprocess
    import sys

    import numpy as np

    cfg = CFG_B
    mdir, out = tmp_path / "m", tmp_path / "out"
    w = write_model(str(mdir), cfg, seed=2)
    a, b = toks(20, cfg["vocab"], 60), toks(5, cfg["vocab"], 61)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:18], "want": [0, 17]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[18:19], "want": []},
                                     {"id": "b", "tokens": b, "want": [4]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[19:], "want": [0]}], "end": ["a"]}]
    exe = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bin", "trace_run")
    r = subprocess.run([sys.executable, exe, "--model", str(mdir), "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    la, lb = O.forward(cfg, w, a), O.forward(cfg, w, b)
    rd = lambda n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
    check(rd(0), la[[0, 17]])
    check(rd(1), lb[[4]])
    check(rd(2), la[[19]])
