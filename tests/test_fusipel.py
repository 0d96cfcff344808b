"""Fusipel through the engine (scheduler, paged pools, model runner, ops)
against the plain float64 oracle in tests/fusipel_oracle.py.

Every test writes its own small checkpoint (config.json + safetensors with
random bf16 weights) and loads it like a served model. The engine runs in
fp32 here so that a structural fault — a key one position off at a window's
edge, a block used twice, a pass reading another pass's pool, a sink left
out — shows far above the rounding floor; one test repeats the comparison
in bf16. Windows are a few tokens wide, so every key inside one carries
weight and a window that is one token off moves the logits visibly.
"""
import io
import json
import math
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import fusipel_oracle as oracle  # noqa: E402

from gpustack_amd.engine import EngineConfig, LLMEngine, SamplingParams  # noqa: E402
from gpustack_amd.engine.config import ModelSpec, RotarySpec  # noqa: E402


def make_engine(model_dir, dtype="float32", blocks=48, max_seqs=4,
                device="cpu", **kw):
    kw.setdefault("max_prefill_tokens", 4096)
    cfg = EngineConfig(model=model_dir, dtype=dtype, device=device,
                       enforce_random_weights=False, kv_cache_blocks=blocks,
                       max_num_seqs=max_seqs, max_model_len=4096, **kw)
    return LLMEngine(cfg)


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def replay(eng, prompts, schedule):
    """schedule: steps, each a list of (request, count). Every position's
    logits are asked for; requests end when their tokens run out. Returns
    request -> [T, vocab]."""
    at = {r: 0 for r in prompts}
    got = {r: [] for r in prompts}
    for step in schedule:
        entries, end = [], []
        for r, n in step:
            lo, hi = at[r], at[r] + n
            entries.append((r, prompts[r][lo:hi], list(range(n))))
            at[r] = hi
            if hi == len(prompts[r]):
                end.append(r)
        logits = eng.replay_step(entries, end)
        off = 0
        for r, n in step:
            got[r].append(logits[off:off + n].double().cpu())
            off += n
    return {r: torch.cat(v) for r, v in got.items() if v}


def err(got, ref):
    """Centred RMS difference relative to the RMS of the reference."""
    d = got.double() - ref
    d = d - d.mean(-1, keepdim=True)
    c = ref - ref.mean(-1, keepdim=True)
    return float((d.pow(2).mean(-1).sqrt() / c.pow(2).mean(-1).sqrt()).max())


TOL = 2e-4      # fp32 engine against the float64 oracle


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = oracle.make_config()
    w = oracle.make_weights(cfg, seed=3)
    d = oracle.save_model(tmp_path_factory.mktemp("fusipel"), cfg, w)
    return cfg, w, d


# ---- configuration ------------------------------------------------------------

def test_config_is_read_from_the_file(model):
    cfg, _, d = model
    spec = ModelSpec.from_dir(d)
    assert spec.architecture == "Fusipel"
    assert spec.vocab_size == cfg["vocab"] and spec.hidden_size == cfg["width"]
    assert spec.residual_multiplier == cfg["residual_mult"]
    assert [i for i, _ in spec.layer_runs()] == [i for i, _ in oracle.layer_order(cfg)]
    assert spec.layer_runs() == oracle.layer_order(cfg)
    m0, m1 = spec.layers[0].mixer, spec.layers[1].mixer
    c0, c1 = cfg["layers"][0]["mixer"], cfg["layers"][1]["mixer"]
    assert (m0.sink, m0.tied_values, m0.qk_norm_full, m0.maps) == (True, True, True, 1)
    assert (m1.maps, m1.window, m1.keep_first, m1.diff) == (
        2, c1["mask"]["size"], c1["mask"]["keep_first"], c1["diff"])
    assert (m0.heads, m0.kv_heads, m0.qk_dim) == (c0["heads"], c0["kv_heads"], c0["dim"])
    # one pool pair per layer RUN, sized by that layer's mixer
    pools = spec.kv_pool_widths()
    assert len(pools) == len(oracle.layer_order(cfg))
    assert pools[1] == ("kv", c1["kv_heads"], 2 * c1["dim"], c1["vdim"])
    assert pools[0] == ("kv", c0["kv_heads"], c0["dim"], c0["dim"])


@pytest.mark.parametrize("rot", [
    {"dims": 8, "base": 10000.0},
    {"dims": 16, "base": 500.0,
     "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}},
    {"dims": 6, "base": 20.0,
     "scaling": {"factor": 2.5, "low": 2.0, "high": 4.0, "original": 30}},
])
def test_rotary_frequencies(rot):
    sc = rot.get("scaling")
    spec = RotarySpec(dims=rot["dims"], base=rot["base"],
                      scaling=(sc["factor"], sc["low"], sc["high"],
                               sc["original"]) if sc else None)
    ref = oracle.rot_freqs(rot)
    got = torch.tensor(spec.inv_freq(), dtype=torch.float64)
    assert torch.allclose(got, ref, rtol=1e-12, atol=0)
    if sc:   # the three branches are all exercised by these parameters
        waves = 2 * math.pi / torch.tensor(
            [rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(rot["dims"] // 2)])
        assert (waves < sc["original"] / sc["high"]).any()
        assert (waves > sc["original"] / sc["low"]).any()


# ---- each mechanism alone -----------------------------------------------------

def test_rotation_and_whole_row_norm_alone():
    """ops.rotary_norm_store against the oracle's pair rotation and unit
    RMS: partial rotation, scaled frequencies, positions in the thousands."""
    from gpustack_amd import ops

    T, H, G, d, eps = 9, 3, 1, 10, 1e-5
    rot = oracle.rot(6, base=30.0)
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(T, (H + G) * d, generator=g)
    qw, kw = torch.rand(H * d, generator=g) + 0.5, torch.rand(G * d, generator=g) + 0.5
    pos = torch.tensor([0, 1, 2, 17, 100, 999, 1000, 2047, 5000], dtype=torch.int32)
    inv = torch.tensor(RotarySpec(dims=6, base=30.0, scaling=(3.0, 1.0, 3.0, 40.0)
                                  ).inv_freq(), dtype=torch.float64).float()
    kc = torch.zeros(T, G, 16, d)
    vc = torch.zeros(T, G, d, 16)
    slots = torch.arange(T) * 16 + 3
    q = torch.empty(T, H * d)
    ops.rotary_norm_store(q, qkv, H * d, G * d, qw, kw, inv, pos, d, kc, vc,
                          slots, eps, True)
    x = qkv.double()
    rq = oracle.rotate_pairs(oracle.unit_rms(x[:, :H * d], eps, qw.double())
                             .view(T, H, d), rot, pos)
    rk = oracle.rotate_pairs(oracle.unit_rms(x[:, H * d:], eps, kw.double())
                             .view(T, G, d), rot, pos)
    assert (q.double().view(T, H, d) - rq).abs().max() < 1e-5
    assert (kc[:, :, 3].double() - rk).abs().max() < 1e-5
    assert torch.equal(vc[:, :, :, 3], qkv[:, H * d:].view(T, G, d))   # raw keys


def test_sink_softmax_and_visibility_alone():
    """ops.paged_attention (one sequence, pages in a shuffled pool) against
    the oracle's visibility matrix and sink softmax."""
    from gpustack_amd import ops

    T, H, G, d, dv, window, keep = 45, 4, 2, 6, 5, 9, 3
    g = torch.Generator().manual_seed(8)
    q = torch.randn(T, H, d, generator=g)
    k = torch.randn(T, G, d, generator=g)
    v = torch.randn(T, G, dv, generator=g)
    sinks = torch.randn(H, generator=g) * 2
    blocks = [4, 1, 3]
    kc, vc = torch.zeros(5, G, 16, d), torch.zeros(5, G, dv, 16)
    for t in range(T):
        kc[blocks[t // 16], :, t % 16] = k[t]
        vc[blocks[t // 16], :, :, t % 16] = v[t]
    bt = torch.tensor([blocks], dtype=torch.int32)
    pos = torch.arange(T, dtype=torch.int32)
    for win, kp, sk in ((window, keep, None), (0, 0, sinks), (window, 0, sinks)):
        out = torch.zeros(T, H, dv)
        ops.paged_attention(out, q, kc, vc, bt, torch.zeros(T, dtype=torch.int32),
                            pos, 0.4, window=win, keep_first=kp, sinks=sk)
        ok = oracle.visible(T, win, kp)
        for a in range(H):
            s = (q[:, a].double() @ k[:, a // 2].double().T) * 0.4
            s = s.masked_fill(~ok, float("-inf"))
            ref = oracle.softmax_with_sink(
                s, None if sk is None else sk[a].double()) @ v[:, a // 2].double()
            assert (out[:, a].double() - ref).abs().max() < 1e-5

def _one(tmp_path, layers, loop=None, mult=0.7, n=37, seed=0, width=20,
         steps=None, **kw):
    cfg = oracle.make_config(width=width, layers=layers, loop=loop, mult=mult)
    w = oracle.make_weights(cfg, seed=seed, **kw)
    d = oracle.save_model(tmp_path, cfg, w)
    toks = tokens_for(cfg, n, seed + 1)
    eng = make_engine(d)
    got = replay(eng, {"a": toks}, steps or [[("a", n)]])["a"]
    return err(got, oracle.forward(cfg, w, toks))


def test_tied_sink_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.tied_layer(ff=0)]) < TOL


def test_large_sinks(tmp_path):
    """Large sinks: dropping one, multiplying it by the score scale or
    adding it once per key would move the output far beyond the tolerance."""
    assert _one(tmp_path, [oracle.tied_layer(ff=0, heads=4, kv_heads=1)],
                sink_gain=4.0) < TOL


def test_diff_window_mixer_alone(tmp_path):
    assert _one(tmp_path, [oracle.diff_layer(ff=0)]) < TOL


def test_gated_feed_forward_and_sandwich_norms(tmp_path):
    assert _one(tmp_path, [oracle.tied_layer(heads=1, kv_heads=1, ff=33)],
                mult=1.3) < TOL


@pytest.mark.parametrize("loop", [(0, 2, 3), (1, 2, 2), (0, 3, 1), (2, 3, 4)])
def test_layer_loop(tmp_path, loop):
    """Passes share weights but not pools; the embedding output re-enters
    before every pass but the first."""
    layers = [oracle.tied_layer(ff=12), oracle.diff_layer(ff=0),
              oracle.tied_layer(heads=2, kv_heads=1, dim=6, rot_dims=2, ff=0)]
    assert _one(tmp_path, layers, loop=loop, n=23,
                steps=[[("a", 9)], [("a", 14)]]) < TOL


@pytest.mark.parametrize("layers", [
    # kv heads == heads in the windowed mixer, value size == score size
    [oracle.diff_layer(heads=2, kv_heads=2, dim=8, vdim=8, window=3,
                       keep_first=1, rot_dims=8)],
    # one kv head for all heads, full rotation, window of one key
    [oracle.diff_layer(heads=6, kv_heads=1, dim=4, vdim=3, window=1,
                       keep_first=0, rot_dims=4),
     oracle.tied_layer(heads=4, kv_heads=1, dim=6, rot_dims=6)],
    # window wider than the sequence, many kept keys
    [oracle.diff_layer(window=500, keep_first=9),
     oracle.tied_layer(heads=5, kv_heads=5, dim=4, rot_dims=2)],
    # more kept keys than the window holds
    [oracle.diff_layer(window=2, keep_first=11, diff=0.8)],
])
def test_other_sizes(tmp_path, layers):
    assert _one(tmp_path, layers, loop=None, n=41, mult=1.0, width=28,
                steps=[[("a", 17)], [("a", 2)], [("a", 21)], [("a", 1)]]) < TOL


def test_no_rotation_and_no_scaling(tmp_path):
    a, b = oracle.diff_layer(), oracle.tied_layer()
    a["mixer"]["rot"] = {"dims": 0, "base": 10.0}
    b["mixer"]["rot"] = {"dims": 4, "base": 7.0}        # no "scaling" key
    assert _one(tmp_path, [a, b], n=19) < TOL


# ---- schedules --------------------------------------------------------------------

def test_whole_prompts_and_first_tokens(model):
    cfg, w, d = model
    eng = make_engine(d)
    for n in (1, 2, 3, 16, 17, 50):
        toks = tokens_for(cfg, n, n)
        got = replay(eng, {"a": toks}, [[("a", n)]])["a"]
        assert err(got, oracle.forward(cfg, w, toks)) < TOL, n


def test_prefill_equals_token_by_token(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 45, 7)
    ref = oracle.forward(cfg, w, toks)
    eng = make_engine(d)
    one = replay(eng, {"a": toks}, [[("a", 1)] for _ in toks])["a"]
    whole = replay(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    assert err(one, ref) < TOL and err(whole, ref) < TOL
    assert err(one, whole.double()) < TOL


@pytest.mark.parametrize("sizes", [
    [2, 2, 2, 3, 2, 30, 1, 1, 2],
    [15, 1, 16, 17, 1, 1],
    [7, 7, 7, 7, 7, 7, 7, 1, 1, 1],
    [33, 2, 16, 1],
])
def test_portions(model, sizes):
    """Portions cut inside pages and inside the windows (5 and 7 keys)."""
    cfg, w, d = model
    toks = tokens_for(cfg, sum(sizes), 11)
    eng = make_engine(d)
    got = replay(eng, {"a": toks}, [[("a", n)] for n in sizes])["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


def test_unequal_batch_equals_each_alone(model):
    cfg, w, d = model
    prompts = {"a": tokens_for(cfg, 40, 1), "b": tokens_for(cfg, 9, 2),
               "c": tokens_for(cfg, 27, 3), "d": tokens_for(cfg, 2, 4)}
    schedule = [
        [("a", 18), ("b", 2)],
        [("a", 1), ("b", 5), ("c", 20)],
        [("a", 1), ("c", 1), ("d", 2)],
        [("b", 1), ("a", 17), ("c", 3)],
        [("c", 1), ("a", 1), ("b", 1)],
        [("a", 2), ("c", 2)],
    ]
    eng = make_engine(d)
    got = replay(eng, prompts, schedule)
    for r, toks in prompts.items():
        assert err(got[r], oracle.forward(cfg, w, toks)) < TOL, r
    alone = make_engine(d)
    for r, toks in prompts.items():
        g = replay(alone, {r: toks}, [[(r, len(toks))]])[r]
        assert err(got[r], g.double()) < TOL, r


def test_blocks_and_slots_are_used_again(model):
    """A pool of 7 usable blocks: every request takes blocks that an ended
    one has just given back, in another order."""
    cfg, w, d = model
    eng = make_engine(d, blocks=8)
    free0 = eng.scheduler.kv.allocator.num_free
    prompts = {f"r{i}": tokens_for(cfg, n, 20 + i)
               for i, n in enumerate([50, 33, 17, 60, 40, 31])}
    schedule = [
        [("r0", 30), ("r1", 2)], [("r0", 20), ("r1", 31)],      # r0, r1 end
        [("r2", 16), ("r3", 40)], [("r2", 1), ("r3", 20)],      # r2, r3 end
        [("r4", 38), ("r5", 2)], [("r4", 2), ("r5", 29)],
    ]
    got = replay(eng, prompts, schedule)
    for r, toks in prompts.items():
        assert err(got[r], oracle.forward(cfg, w, toks)) < TOL, r
    assert eng.scheduler.kv.allocator.num_free == free0


def test_long_decoding_across_pages_and_windows(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 5 + 140, 13)
    eng = make_engine(d)
    got = replay(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 140)["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < TOL


def test_bf16_engine_is_close(model):
    cfg, w, d = model
    toks = tokens_for(cfg, 40, 5)
    eng = make_engine(d, dtype="bfloat16")
    got = replay(eng, {"a": toks}, [[("a", 23)], [("a", 16)], [("a", 1)]])["a"]
    assert err(got, oracle.forward(cfg, w, toks)) < 0.12


# ---- faults that random weights would hide ------------------------------------------------

def standout_model(tmp_path, far_pos, n, window=0, keep_first=0, kind="tied"):
    """A one-mixer model in which the LAST token's query matches the key at
    `far_pos` far better than any other. W_k is W_q with its input channels
    shifted by one and the token at far_pos has the last token's embedding
    shifted back, so k(far) = q(last) up to the few rotated channels, while
    the last token's own key (and every other) is unrelated. One score
    stands out among n: losing that key, or wrongly admitting it, changes
    the row wholly."""
    if kind == "tied":
        L = oracle.tied_layer(heads=2, kv_heads=2, dim=32, rot_dims=2, ff=0,
                              scale=0.5)
    else:
        L = oracle.diff_layer(heads=2, kv_heads=2, dim=32, vdim=6, rot_dims=2,
                              window=window, keep_first=keep_first, ff=0,
                              scale=0.35)
    cfg = oracle.make_config(width=32, vocab=40, layers=[L], loop=None)
    w = oracle.make_weights(cfg, seed=9)
    w["l0.norm1"] = torch.ones_like(w["l0.norm1"])
    w["l0.mix.k"] = torch.roll(w["l0.mix.q"], -1, dims=1).contiguous()
    w["l0.mix.k.b"] = w["l0.mix.q.b"].clone()
    if kind == "tied":
        w["l0.mix.k.norm"] = w["l0.mix.q.norm"].clone()
    w["embed"][38] = torch.roll(w["embed"][39], -1, dims=0)
    toks = [t % 38 for t in tokens_for(cfg, n, 5)]
    toks[far_pos] = 38
    toks[-1] = 39
    return cfg, w, oracle.save_model(tmp_path, cfg, w), toks


@pytest.mark.parametrize("far_pos", [0, 15, 16, 31, 200])
@pytest.mark.parametrize("decode", [False, True])
def test_far_key_among_hundreds(tmp_path, far_pos, decode):
    cfg, w, d, toks = standout_model(tmp_path, far_pos, 420)
    ref = oracle.forward(cfg, w, toks)[-1:]
    # the key matters: without it the last row is another one altogether
    other = list(toks)
    other[far_pos] = 1
    assert err(oracle.forward(cfg, w, other)[-1:], ref) > 0.05
    eng = make_engine(d)
    n = len(toks)
    steps = [[("a", n - 1)], [("a", 1)]] if decode else [[("a", n)]]
    got = replay(eng, {"a": toks}, steps)["a"][-1:]
    assert err(got, ref) < TOL


@pytest.mark.parametrize("gap", [-1, 0, 1])   # just inside, at, just outside
@pytest.mark.parametrize("decode", [False, True])
@pytest.mark.parametrize("edge", ["window", "first"])
def test_window_and_kept_keys_edges(tmp_path, gap, decode, edge):
    n, window, keep = 83, 19, 4
    if edge == "window":
        far_pos = (n - 1) - (window - 1) - gap    # gap <= 0: seen
    else:
        far_pos = keep - 1 + gap                  # gap <= 0: kept
    cfg, w, d, toks = standout_model(tmp_path, far_pos, n, window, keep,
                                     kind="diff")
    ref = oracle.forward(cfg, w, toks)[-1:]
    eng = make_engine(d)
    steps = [[("a", n - 1)], [("a", 1)]] if decode else [[("a", 40)], [("a", n - 40)]]
    got = replay(eng, {"a": toks}, steps)["a"][-1:]
    assert err(got, ref) < TOL
    # and the edge is where the oracle says: moving the mask by one key
    # changes this row
    moved = json.loads(json.dumps(cfg))
    mk = moved["layers"][0]["mixer"]["mask"]
    if edge == "window":
        mk["size"] += 1 if gap == 1 else -1 if gap == 0 else 0
    else:
        mk["keep_first"] += 1 if gap == 1 else -1 if gap == 0 else 0
    if gap != -1:
        assert err(oracle.forward(moved, w, toks)[-1:], ref) > 0.02


# ---- the framework's own entry points -----------------------------------------------------

def test_greedy_generation_through_the_scheduler(model):
    cfg, w, d = model
    eng = make_engine(d)
    prompts = [tokens_for(cfg, n, 40 + n) for n in (3, 21, 9)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=14, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 14)


def test_generation_with_chunked_prefill_and_small_pool(model):
    cfg, w, d = model
    eng = make_engine(d, blocks=14, max_prefill_tokens=16)
    prompts = [tokens_for(cfg, n, 60 + n) for n in (45, 7, 30)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 10)


def test_replay_command(model, tmp_path):
    """The replay driver writes the wanted rows, step by step."""
    from gpustack_amd.engine.replay import run_trace

    cfg, w, d = model
    toks = tokens_for(cfg, 30, 77)
    lines = [json.dumps({"step": 0, "entries": [
                {"id": "x", "tokens": toks[:20], "want": [0, 19]}], "end": []}),
             json.dumps({"step": 1, "entries": [
                 {"id": "x", "tokens": toks[20:29], "want": []}], "end": []}),
             json.dumps({"step": 2, "entries": [
                 {"id": "x", "tokens": toks[29:], "want": [0]}], "end": ["x"]})]
    out = io.StringIO()
    assert run_trace(d, "float32", str(tmp_path / "o"), 64, lines=lines,
                     out=out, device="cpu") == 0
    assert out.getvalue().split() == ["done", "0", "done", "1", "done", "2"]
    import numpy as np

    ref = oracle.forward(cfg, w, toks)
    a = torch.from_numpy(np.fromfile(tmp_path / "o" / "0.f32", dtype="<f4")
                         ).view(2, -1)
    b = torch.from_numpy(np.fromfile(tmp_path / "o" / "2.f32", dtype="<f4")
                         ).view(1, -1)
    assert not (tmp_path / "o" / "1.f32").exists()
    assert err(a, ref[[0, 19]]) < TOL and err(b, ref[[29]]) < TOL
