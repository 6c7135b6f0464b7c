"""Medilix family on the CPU path (fp32) against the plain float64 oracle in
tests/medilix_oracle.py: every mechanism alone, then whole models through the
engine's segment step, cache / slot reuse, and greedy generation through
generate() and the scheduler. Configurations are small and lopsided: value
sizes that differ from key sizes, grouped and ungrouped heads, odd decay
ranks, a loop that starts after the first layer, layers without a
feed-forward, one norm group and several, routers with and without identity
experts, groups and negative corrections."""

import json
import os

import pytest
import torch

import medilix_oracle as O
from kllms_amd.engine.config import (EngineConfig, GluSpec, MaskedAttnSpec, MlstmSpec, RoutedExpertsSpec, WkvSpec)
from kllms_amd.engine.engine import GenRequest, LLMEngine
from kllms_amd.engine.kvcache import HybridStateCache, LayerCacheSpec
from kllms_amd.engine.sampling import SamplingParams
from kllms_amd.engine.scheduler import BatchScheduler
from kllms_amd.models.llama import ForwardBatch
from kllms_amd.models.mixers import ClampedGLU, MlstmMixer, RoutedExperts, WindowSinkAttention, WkvMixer
from kllms_amd import ops

EPS = 1e-5


def attn(heads=4, kv=2, dim=8, vdim=12, size=9, keep=3, scale=1.0, mlp="dense"):
    return {"type": "attention", "mlp": MLPS[mlp],
            "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                      "mask": {"size": size, "keep_first": keep}}}


def wkv(heads=3, dim=8, mlp="moe"):
    return {"type": "wkv", "mixer": {"heads": heads, "dim": dim}, "mlp": MLPS[mlp]}


def mlstm(heads=2, dim=6, vdim=10, cap=15.0, mlp="moe"):
    return {"type": "mlstm", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "gate_cap": cap}, "mlp": MLPS[mlp]}


MLPS = {
    None: None,
    "dense": {"kind": "dense", "ff": 40, "limit": 0.8},
    "moe": {"kind": "moe", "expert": {"ff": 20},
            "router": {"experts": 6, "identity": 3, "top": 2, "groups": {"count": 3, "keep": 2}}},
    "moe_plain": {"kind": "moe", "expert": {"ff": 12},
                  "router": {"experts": 4, "identity": 0, "top": 1, "groups": {"count": 1, "keep": 1}}},
}

BIGRAM = {"buckets": 23, "mul_prev": 13, "mul_cur": 3}
# loop over the middle layers, three passes
CFG_A = {"architecture": "Medilix", "vocab": 61, "width": 24, "norm": {"eps": EPS, "groups": 3},
         "embedding": {"scale": 5.0, "bigram": BIGRAM},
         "layers": [attn(), wkv(), mlstm(), attn(heads=2, kv=2, dim=4, vdim=4, size=5, keep=0, mlp="moe")],
         "loop": {"start": 1, "stop": 3, "times": 3}}
# one norm group, heads not grouped, no identity experts, top 1, layers without a feed-forward,
# a loop of one pass from the first layer, a window longer than every test prompt
CFG_B = {"architecture": "Medilix", "vocab": 47, "width": 20, "norm": {"eps": 1e-6, "groups": 1},
         "embedding": {"scale": 1.0, "bigram": {"buckets": 7, "mul_prev": 1, "mul_cur": 1}},
         "layers": [mlstm(heads=1, dim=4, vdim=4, cap=2.0, mlp=None), wkv(heads=1, dim=12, mlp="dense"),
                    attn(heads=3, kv=3, dim=6, vdim=2, size=500, keep=1, scale=0.4, mlp="moe_plain"),
                    wkv(heads=5, dim=4, mlp=None)],
         "loop": {"start": 0, "stop": 2, "times": 1}}
# no loop at all
CFG_C = {"architecture": "Medilix", "vocab": 33, "width": 16, "norm": {"eps": EPS, "groups": 2},
         "embedding": {"scale": 2.0, "bigram": BIGRAM},
         "layers": [wkv(heads=2, dim=8, mlp="dense"), attn(heads=2, kv=1, dim=8, vdim=8, size=4, keep=2)],
         "loop": None}


def write_model(tmp, cfg, seed=0, decay_rank=5):
    from safetensors.torch import save_file

    w = O.random_weights(cfg, seed, decay_rank)
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
    d = tmp_path_factory.mktemp("med_a")
    w = write_model(str(d), CFG_A, seed=1)
    return CFG_A, w, make_engine(d, blocks=96)


@pytest.fixture(scope="module")
def model_b(tmp_path_factory):
    d = tmp_path_factory.mktemp("med_b")
    w = write_model(str(d), CFG_B, seed=2, decay_rank=3)
    return CFG_B, w, make_engine(d, blocks=40, slots=3)


def toks(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def check(got, want, atol=2e-4):
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=atol)


# --- mechanisms alone -----------------------------------------------------------

def seg_batch(cache, seqs, counts):
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


def run_mixer(mod, h, cuts, page=4):
    """Feed h [L, W] through a mixer in portions; the sequence does not get
    slot 0 and its pages are not the first ones."""
    cache = HybridStateCache([mod.cache_spec()], page, 200, 3, "cpu", torch.float32)
    cache.slots.alloc()
    for _ in range(3):
        cache.allocator.alloc()
    seq = cache.open_sequence()
    outs, at = [], 0
    for n in cuts:
        outs.append(mod(h[at:at + n].float(), seg_batch(cache, [seq], [n]), cache.layer_caches()[0]))
        at += n
    return torch.cat(outs)


def load_module(mod, w, pre):
    for name, dst in mod.checkpoint_map(pre).items():
        dst.copy_(w[name].to(dst.dtype))


def one_layer(layer, width=24, seed=3, decay_rank=5):
    cfg = {"vocab": 8, "width": width, "norm": {"eps": EPS, "groups": 1}, "layers": [layer]}
    return O.random_weights(cfg, seed, decay_rank)


def rows(L, W, seed):
    return torch.randn(L, W, generator=torch.Generator().manual_seed(seed), dtype=torch.float64)


CUTS = [[60], [70], [25] + [1] * 35, [2, 5, 16, 1, 2, 17, 3, 14], [9, 2, 10, 1, 38]]


@pytest.mark.parametrize("cuts", CUTS)
def test_window_attention_edges(cuts):
    """Window 9 + 3 kept first tokens on 4-token pages: with unit-norm q and k
    and a scale of 1 single keys dominate the softmax, so a window, a kept
    run or a page border that is one position off shows at once."""
    layer = attn(size=9, keep=3, scale=1.0)
    w = one_layer(layer)
    m = layer["mixer"]
    mod = WindowSinkAttention(MaskedAttnSpec(heads=4, kv_heads=2, dim=8, vdim=12, scale=1.0, mask_size=9,
                                             keep_first=3), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    h = rows(sum(cuts), 24, 4)
    check(run_mixer(mod, h, cuts), O.attention(h, w, "l0.mix.", m, EPS))


def test_window_kept_tokens_and_sink_are_visible():
    """What the comparison above rests on: in the oracle, a key just inside
    the window or among the kept first tokens changes the output, one just
    outside does not, and the sink takes weight."""
    layer = attn(size=9, keep=3, scale=1.0)
    w = one_layer(layer)
    m = layer["mixer"]
    a = rows(30, 24, 5)

    def out_at(i, changed):
        b = a.clone()
        b[changed] = rows(1, 24, 99)[0]
        return O.attention(b, w, "l0.mix.", m, EPS)[i], O.attention(a, w, "l0.mix.", m, EPS)[i]

    for i, j, seen in [(20, 12, True), (20, 11, False), (20, 2, True), (20, 3, False), (8, 0, True), (12, 3, False)]:
        x, y = out_at(i, j)
        assert (float((x - y).abs().max()) > 1e-6) == seen, (i, j)
    # a sequence of one token: every head's weight is e / (1 + e), not 1
    h = a[:1]
    W = lambda n: w["l0.mix." + n].double()
    q = O.rms_plain((h @ W("q").T).reshape(4, 8), EPS) * W("q.norm")
    k = O.rms_plain((h @ W("k").T).reshape(2, 8), EPS) * W("k.norm")
    v = (h @ W("v").T).reshape(2, 12)
    heads = []
    for hh in range(4):
        e = torch.exp((q[hh] * k[hh // 2]).sum() * m["scale"])
        assert 0.0 < float(e / (1 + e)) < 1.0
        heads.append(e / (1 + e) * v[hh // 2])
    want = (torch.cat(heads) * torch.sigmoid(h @ W("g").T)[0]) @ W("o").T
    check(O.attention(h, w, "l0.mix.", m, EPS)[0], want, atol=1e-9)
    mod = WindowSinkAttention(MaskedAttnSpec(heads=4, kv_heads=2, dim=8, vdim=12, scale=1.0, mask_size=9,
                                             keep_first=3), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    check(run_mixer(mod, h, [1])[0], want)


@pytest.mark.parametrize("cuts", CUTS)
@pytest.mark.parametrize("rank", [5, 1])
def test_wkv_mixer(cuts, rank):
    layer = wkv(heads=3, dim=8)
    w = one_layer(layer, decay_rank=rank)
    mod = WkvMixer(WkvSpec(heads=3, dim=8, decay_rank=rank), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    h = rows(sum(cuts), 24, 6)
    check(run_mixer(mod, h, cuts), O.wkv(h, w, "l0.mix.", layer["mixer"], EPS))


def test_wkv_reaches_far_back():
    """With slow decays the first token still moves the output 50 tokens later."""
    layer = wkv(heads=3, dim=8)
    w = one_layer(layer)
    w["l0.mix.w0"] = torch.full_like(w["l0.mix.w0"], -6.0)
    a = rows(52, 24, 7)
    b = a.clone()
    b[0] *= -1.0
    ya, yb = (O.wkv(x, w, "l0.mix.", layer["mixer"], EPS)[51] for x in (a, b))
    assert float((ya - yb).abs().max()) > 1e-4
    mod = WkvMixer(WkvSpec(heads=3, dim=8, decay_rank=5), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    check(run_mixer(mod, a, [40] + [1] * 12), O.wkv(a, w, "l0.mix.", layer["mixer"], EPS))


@pytest.mark.parametrize("cuts", CUTS)
@pytest.mark.parametrize("cap", [15.0, 1.5])
def test_mlstm_mixer(cuts, cap):
    layer = mlstm(heads=2, dim=6, vdim=10, cap=cap)
    w = one_layer(layer)
    mod = MlstmMixer(MlstmSpec(heads=2, dim=6, vdim=10, gate_cap=cap), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    h = rows(sum(cuts), 24, 8) * 2.0
    check(run_mixer(mod, h, cuts), O.mlstm(h, w, "l0.mix.", layer["mixer"], EPS))


def test_mlstm_running_maximum_starts_at_zero():
    """Strongly negative input gates: a maximum that started at minus infinity
    would rescale the first updates to 1 and change the output."""
    layer = mlstm(heads=2, dim=6, vdim=10)
    w = one_layer(layer)
    w["l0.mix.i.b"] = torch.full_like(w["l0.mix.i.b"], -8.0)
    mod = MlstmMixer(MlstmSpec(heads=2, dim=6, vdim=10, gate_cap=15.0), 24, EPS, torch.float32)
    load_module(mod, w, "l0.mix.")
    h = rows(12, 24, 9)
    check(run_mixer(mod, h, [5, 1, 6]), O.mlstm(h, w, "l0.mix.", layer["mixer"], EPS), atol=1e-5)


def test_clamped_glu_both_clamps_active():
    mlp = MLPS["dense"]
    w = O.random_weights({"vocab": 8, "width": 24, "norm": {"eps": EPS, "groups": 1},
                          "layers": [dict(wkv(), mlp=mlp)]}, 3)
    h = rows(40, 24, 10) * 2
    g = h @ w["l0.mlp.gate"].double().T
    u = h @ w["l0.mlp.up"].double().T
    assert (g > 0.8).any() and (u > 0.8).any() and (u < -0.8).any()
    mod = ClampedGLU(GluSpec(ff=40, limit=0.8), 24, torch.float32)
    load_module(mod, w, "l0.mlp.")
    check(mod(h.float()), O.dense_ff(h, w, "l0.mlp.", mlp))


@pytest.mark.parametrize("name,T,sorted_form", [("moe", 7, False), ("moe", 90, True), ("moe", 33, True),
                                               ("moe_plain", 5, False), ("moe_plain", 70, True)])
def test_routed_experts(name, T, sorted_form, monkeypatch):
    """Both forms (every expert on every row; rows sorted by expert) against
    the per-token oracle; corrections are negative, so an excluded group must
    count as minus infinity, not 0."""
    if sorted_form:
        monkeypatch.setattr(RoutedExperts, "DENSE_MAX_ROWS", 0)
    mlp = MLPS[name]
    r = mlp["router"]
    w = O.random_weights({"vocab": 8, "width": 24, "norm": {"eps": EPS, "groups": 1},
                          "layers": [dict(wkv(), mlp=mlp)]}, 11)
    n = r["experts"] + r["identity"]
    w["l0.mlp.correction"] = (-0.3 - 0.2 * torch.rand(n, generator=torch.Generator().manual_seed(5))).bfloat16().float()
    mod = RoutedExperts(RoutedExpertsSpec(experts=r["experts"], identity=r["identity"], top=r["top"],
                                          group_count=r["groups"]["count"], group_keep=r["groups"]["keep"],
                                          ff=mlp["expert"]["ff"]), 24, torch.float32)
    load_module(mod, w, "l0.mlp.")
    h = rows(T, 24, 12)
    check(mod(h.float()), O.moe_ff(h, w, "l0.mlp.", mlp))
    if r["identity"]:
        z = h @ w["l0.mlp.router"].double().T
        picks = [O.route(z[t], w["l0.mlp.correction"].double(), r["top"], r["groups"]["count"],
                         r["groups"]["keep"])[0] for t in range(T)]
        assert any(e >= r["experts"] for p in picks for e in p) and any(e < r["experts"] for p in picks for e in p)


def test_router_groups_limit_the_choice():
    z = torch.tensor([[0.0, 3.0, 0.1, 0.2, 2.9, 2.8]])
    corr = torch.zeros(6)
    idx, wt = ops.moe_route(z, corr, 2, 3, 1)
    # groups {0,1} {2,3} {4,5}: the first has the largest member, so both picks come from it,
    # although 4 and 5 score higher than 0
    assert sorted(idx[0].tolist()) == [0, 1]
    chosen, ws = O.route(z[0].double(), corr.double(), 2, 3, 1)
    assert sorted(chosen) == sorted(idx[0].tolist())
    torch.testing.assert_close(wt[0].double().sort().values, torch.tensor(ws, dtype=torch.float64).sort().values,
                               rtol=1e-5, atol=1e-6)


def test_group_norm_and_bigram_rows():
    x = rows(5, 24, 13)
    wt = rows(1, 24, 14)[0]
    h1, _ = ops.group_norm_pair(x.float().clone(), None, None, wt.float(), None, 3, EPS, torch.float32)
    check(h1, O.group_rms(x, wt, 3, EPS))
    cfg = dict(CFG_A, layers=[])
    w = {"embed": rows(61, 24, 15).float(), "bigram": rows(24, 24, 16).float()}
    ids = [7, 7, 60, 0, 5]
    want = O.embed_tokens(ids, w, cfg)
    # the last bucket row is used for the first token only
    check(want[0], w["embed"][7].double() * 5.0 + w["bigram"][23].double())
    i32 = lambda v: torch.tensor(v, dtype=torch.int32)
    state = i32([99, 99])
    a = ops.embed_bigram(torch.tensor(ids[:3]), w["embed"], w["bigram"], 5.0, 13, 3, 23, state, i32([1]), i32([0, 3]),
                         i32([0]), i32([0, 0, 0]))
    b = ops.embed_bigram(torch.tensor(ids[3:]), w["embed"], w["bigram"], 5.0, 13, 3, 23, state, i32([1]), i32([0, 2]),
                         i32([3]), i32([0, 0]))
    check(torch.cat([a, b]), want)
    assert state.tolist() == [99, 5]


# --- whole models through the engine's step function ----------------------------------

def run_cuts(eng, ids, cuts, want_all=True):
    seq = eng.open_sequence()
    outs, at = [], 0
    for n in cuts:
        outs.append(eng.step_segments([(seq, ids[at:at + n], list(range(n)))]))
        at += n
    eng.kv.free_sequence(seq)
    return torch.cat(outs)


def test_whole_prompt_and_first_tokens(model_a):
    cfg, w, eng = model_a
    ids = toks(45, cfg["vocab"], 20)
    want = O.forward(ids, w, cfg)
    check(run_cuts(eng, ids, [45]), want)
    check(run_cuts(eng, ids[:1], [1]), want[:1])
    check(run_cuts(eng, ids[:3], [1, 1, 1]), want[:3])


def test_layer_runs_have_their_own_state(model_a):
    cfg, w, eng = model_a
    assert len(eng.kv.layers) == 1 + 3 * 2 + 1 + 1       # layer runs + the embedding's entry
    ids = toks(12, cfg["vocab"], 21)
    _, layers = O.forward(ids, w, cfg, return_layers=True)
    eng.model.trace_layers = []
    try:
        run_cuts(eng, ids, [12])
        got = eng.model.trace_layers
    finally:
        eng.model.trace_layers = None
    assert len(got) == len(layers) == 8
    for a, b in zip(got, layers):
        check(a, b, atol=5e-4)


def test_prefill_then_decode_long(model_a):
    cfg, w, eng = model_a
    ids = toks(4 + 130, cfg["vocab"], 22)
    check(run_cuts(eng, ids, [4] + [1] * 130), O.forward(ids, w, cfg), atol=5e-4)


@pytest.mark.parametrize("cuts", [[2] * 20, [7, 2, 13, 1, 1, 16], [3, 9, 2, 2, 24], [39, 1]])
def test_portions(model_a, cuts):
    cfg, w, eng = model_a
    ids = toks(sum(cuts), cfg["vocab"], 23)
    check(run_cuts(eng, ids, cuts), O.forward(ids, w, cfg))


def test_mixed_batches_reuse_blocks_and_slots(model_b):
    """Five unequal requests through three slots and a pool smaller than their
    sum: portions beside single tokens, requests that pause, slots and pages
    that change hands."""
    cfg, w, eng = model_b
    reqs = {n: toks(L, cfg["vocab"], 30 + i) for i, (n, L) in enumerate(
        [("a", 70), ("b", 9), ("c", 33), ("d", 2), ("e", 41)])}
    want = {n: O.forward(ids, w, cfg) for n, ids in reqs.items()}
    plan = [[("a", 30), ("b", 2)], [("a", 1), ("b", 6), ("c", 20)], [("c", 1), ("b", 1)],        # b ends
            [("a", 2), ("d", 2), ("c", 12)],                                                   # d, c end
            [("a", 37), ("e", 1)], [("e", 40)]]
    at = {n: 0 for n in reqs}
    live = {}
    for step in plan:
        entries = []
        for n, c in step:
            if n not in live:
                live[n] = eng.open_sequence()
            entries.append((live[n], reqs[n][at[n]:at[n] + c], list(range(c))))
        got = eng.step_segments(entries)
        r = 0
        for n, c in step:
            check(got[r:r + c], want[n][at[n]:at[n] + c])
            r += c
            at[n] += c
            if at[n] == len(reqs[n]):
                eng.kv.free_sequence(live.pop(n))
    assert not live and eng.kv.slots.num_free == 3 and eng.kv.allocator.num_free == eng.kv.num_blocks


def test_slot_state_is_not_inherited(model_b):
    cfg, w, eng = model_b
    a, b = toks(25, cfg["vocab"], 40), toks(11, cfg["vocab"], 41)
    s = eng.open_sequence()
    eng.step_segments([(s, a, [])])
    slot = s.state_slot
    eng.kv.free_sequence(s)
    s2 = eng.open_sequence()
    assert s2.state_slot == slot
    check(eng.step_segments([(s2, b, list(range(11)))]), O.forward(b, w, cfg))
    eng.kv.free_sequence(s2)


def test_no_loop_and_short_window(tmp_path):
    w = write_model(str(tmp_path), CFG_C, seed=3, decay_rank=1)
    eng = make_engine(tmp_path)
    ids = toks(30, CFG_C["vocab"], 42)
    want = O.forward(ids, w, CFG_C)
    check(run_cuts(eng, ids, [30]), want)
    check(run_cuts(eng, ids, [3, 1, 1, 2, 23]), want)


def oracle_greedy(cfg, w, prompt, n):
    ids = list(prompt)
    for _ in range(n):
        ids.append(int(O.forward(ids, w, cfg)[-1].argmax()))
    return ids[len(prompt):]


def test_greedy_generation_and_fork(model_a):
    cfg, w, eng = model_a
    p1, p2 = toks(21, cfg["vocab"], 50), toks(5, cfg["vocab"], 51)
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
        p1, p2 = toks(29, CFG_A["vocab"], 52), toks(6, CFG_A["vocab"], 53)
        sp = lambda n: SamplingParams(temperature=0.0, max_tokens=n)
        f1 = sched.submit(GenRequest(prompt_ids=p1, n=1, sampling=sp(6)))
        f2 = sched.submit(GenRequest(prompt_ids=p2, n=2, sampling=sp(8)))
        o1, o2 = f1.result(timeout=120), f2.result(timeout=120)
    finally:
        sched.shutdown()
    assert o1.streams[0].token_ids == oracle_greedy(CFG_A, w, p1, 6)
    want2 = oracle_greedy(CFG_A, w, p2, 8)
    assert [s.token_ids for s in o2.streams] == [want2, want2]
    assert eng.kv.slots.num_free == eng.kv.slots.num_slots


def test_config_reader_takes_sizes_from_file_and_tensors(tmp_path):
    write_model(str(tmp_path), CFG_B, seed=2, decay_rank=3)
    arch = EngineConfig(model=str(tmp_path)).resolve_arch()
    assert arch.arch == "medilix" and arch.vocab_size == 47 and arch.hidden_size == 20 and arch.norm_groups == 1
    assert arch.layers[1].wkv.decay_rank == 3 and arch.layers[0].mlp is None and arch.layers[0].mlstm.gate_cap == 2.0
    assert arch.layers[2].attention.keep_first == 1 and arch.layers[2].attention.mask_size == 500
    assert (arch.loop.start, arch.loop.stop, arch.loop.times) == (0, 2, 1)
    assert [i for i, _ in arch.layer_runs()] == [0, 1, 2, 3] and arch.layer_runs()[0][1]
    assert arch.bigram.buckets == 7 and arch.layers[2].mlp.identity == 0


def test_presets_build_and_generate():
    eng = LLMEngine(EngineConfig(model="tiny-medilix", dtype="float32", device="cpu", max_kv_blocks=64,
                                 max_state_slots=4, use_hip_graphs=False))
    out = eng.generate([GenRequest(prompt_ids=toks(9, 512, 60), n=2, sampling=SamplingParams(temperature=0.0, max_tokens=5))])
    assert len(out[0].streams) == 2 and out[0].streams[0].token_ids == out[0].streams[1].token_ids


def test_trace_replay_cli(tmp_path):
    import subprocess
    import sys

    import numpy as np

    cfg = CFG_C
    mdir, out = tmp_path / "m", tmp_path / "out"
    w = write_model(str(mdir), cfg, seed=4)
    a, b = toks(20, cfg["vocab"], 61), toks(5, cfg["vocab"], 62)
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
    la, lb = O.forward(a, w, cfg), O.forward(b, w, cfg)
    rd = lambda n: torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(-1, cfg["vocab"]).copy())
    check(rd(0), la[[0, 17]])
    check(rd(1), lb[[4]])
    check(rd(2), la[[19]])
