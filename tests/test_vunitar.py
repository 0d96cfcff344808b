"""Vunitar through the engine (scheduler, paged pool, model runner, ops)
against the plain float64 oracle in tests/vunitar_oracle.py.

Every test writes its own small checkpoint (config.json + safetensors with
random bf16 weights) and loads it like a served model. The engine runs in
fp32 here so that a structural fault — a key one position off at a page
border, a block used twice, a lost previous token — shows far above the
rounding floor; one test repeats the comparison in bf16.
"""
import json
import math
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import vunitar_oracle as oracle  # noqa: E402

from gpustack_amd import ops  # noqa: E402
from gpustack_amd.engine import EngineConfig, LLMEngine, SamplingParams  # noqa: E402

BF = torch.bfloat16


def mixer(heads=3, dim=8, vdim=5, kv_rank=12, scale=None):
    return {"heads": heads, "dim": dim, "vdim": vdim, "kv_rank": kv_rank,
            "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}


def moe(experts=6, top=2, count=3, keep=2, ff=10, scale=1.7, shared=7):
    m = {"kind": "moe", "expert": {"ff": ff},
         "router": {"experts": experts, "top": top, "scale": scale,
                    "groups": {"count": count, "keep": keep}}}
    if shared:
        m["shared"] = {"ff": shared}
    return m


def make_config(width=20, vocab=53, layers=None, bigram=(11, 5, 3), cap=9.0):
    cfg = {"architecture": "Vunitar", "vocab": vocab, "width": width,
           "norm": {"eps": 1e-5},
           "layers": layers or [
               {"type": "latent_attention", "mixer": mixer(),
                "mlp": {"kind": "dense", "ff": 24}},
               {"type": "latent_attention",
                "mixer": mixer(heads=2, dim=6, vdim=9, kv_rank=10),
                "mlp": moe()},
           ]}
    if bigram:
        cfg["embedding"] = {"bigram": {"buckets": bigram[0],
                                       "mul_prev": bigram[1],
                                       "mul_cur": bigram[2]}}
    if cap:
        cfg["logit_softcap"] = cap
    return cfg


def make_weights(cfg, seed=0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(BF)

    def vec(n, base=1.0):
        return (base + 0.2 * torch.randn(n, generator=g)).to(BF)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(BF),
         "final.norm": vec(W), "head": lin(cfg["vocab"], W, 2.0)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        w["bigram"] = torch.randn(bg["buckets"] + 1, W, generator=g).to(BF)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        w[p + "mix.q"] = lin(m["heads"] * m["dim"], W, 2.0)
        w[p + "mix.dkv"] = lin(m["kv_rank"], W)
        w[p + "mix.dkv.norm"] = vec(m["kv_rank"])
        w[p + "mix.uk"] = lin(m["heads"] * m["dim"], m["kv_rank"], 2.0)
        w[p + "mix.uv"] = lin(m["heads"] * m["vdim"], m["kv_rank"])
        w[p + "mix.o"] = lin(W, m["heads"] * m["vdim"])
        w[p + "norm1"], w[p + "ls1"] = vec(W), vec(W, 0.6)
        f = L.get("mlp")
        if not f:
            continue
        w[p + "norm2"], w[p + "ls2"] = vec(W), vec(W, 0.6)
        if f["kind"] == "dense":
            w[p + "mlp.up"], w[p + "mlp.down"] = lin(f["ff"], W), lin(W, f["ff"])
        else:
            r = f["router"]
            w[p + "mlp.router"] = lin(r["experts"], W, 3.0)
            for e in range(r["experts"]):
                w[p + f"mlp.e{e}.up"] = lin(f["expert"]["ff"], W)
                w[p + f"mlp.e{e}.down"] = lin(W, f["expert"]["ff"])
            if f.get("shared"):
                w[p + "mlp.shared.up"] = lin(f["shared"]["ff"], W)
                w[p + "mlp.shared.down"] = lin(W, f["shared"]["ff"])
                w[p + "mlp.shared.sg"] = lin(1, W, 2.0)
    return w


def save_model(path: Path, cfg, weights):
    from safetensors.torch import save_file

    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()},
              str(path / "model.safetensors"))
    return str(path)


def make_engine(model_dir, dtype="float32", blocks=40, max_seqs=4,
                device="cpu", **kw):
    cfg = EngineConfig(model=model_dir, dtype=dtype, device=device,
                       enforce_random_weights=False, kv_cache_blocks=blocks,
                       max_num_seqs=max_seqs, max_model_len=4096,
                       max_prefill_tokens=4096, **kw)
    return LLMEngine(cfg)


def run_schedule(eng, reqs, steps):
    """reqs: id -> tokens; steps: list of [(id, n), ...]. Feeds each request
    n tokens per step, asks for every position, ends a request with its last
    token. Returns id -> logits [T, V]."""
    at = {i: 0 for i in reqs}
    got = {i: [] for i in reqs}
    for step in steps:
        entries, end = [], []
        for i, n in step:
            lo = at[i]
            entries.append((i, reqs[i][lo:lo + n], list(range(n))))
            at[i] = lo + n
            if at[i] == len(reqs[i]):
                end.append(i)
        lg = eng.replay_step(entries, end).cpu()
        off = 0
        for i, n in step:
            got[i].append(lg[off:off + n])
            off += n
    assert all(at[i] == len(reqs[i]) for i in reqs)
    return {i: torch.cat(v) for i, v in got.items()}


def toks(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, want, tol=2e-4):
    d = (got.double() - want).abs().max().item()
    assert d < tol, f"max abs logit difference {d}"


@pytest.fixture(scope="module")
def small(tmp_path_factory):
    cfg = make_config()
    w = make_weights(cfg, seed=1)
    d = save_model(tmp_path_factory.mktemp("vun") / "m", cfg, w)
    return cfg, w, d


# ---- each mechanism alone ---------------------------------------------------

def test_pair_hash_embedding_alone():
    V, W, B = 30, 6, 7
    g = torch.Generator().manual_seed(0)
    emb, pair = torch.randn(V, W, generator=g), torch.randn(B + 1, W, generator=g)
    seq = [4, 29, 29, 0, 17]
    want = oracle.embed_tokens(seq, emb.double(), pair.double(), B, 13, 5)
    x = torch.empty(len(seq), W)
    ops.embed_pair_hash(x, None, torch.tensor(seq), torch.tensor([-1] + seq[:-1]),
                        emb, pair, B, 13, 5)
    close(x, want, 1e-6)
    # the first token reads the extra row, whatever its id
    close(x[0], emb[4].double() + pair[B].double(), 1e-6)


def test_output_norm_with_layer_scale_alone():
    g = torch.Generator().manual_seed(2)
    x, a = torch.randn(5, 14, generator=g), torch.randn(5, 14, generator=g) * 4
    w, s = torch.randn(14, generator=g), torch.randn(14, generator=g)
    want = x.double() + oracle.rms_norm(a.double(), w.double(), 1e-3) * s.double()
    ops.rms_scale_add(x, a, w, s, 1e-3, None)
    close(x, want, 1e-5)


@pytest.mark.parametrize("E,G,keep,top", [(6, 3, 2, 2), (8, 1, 1, 3),
                                          (9, 3, 3, 4), (12, 4, 1, 3)])
def test_group_limited_routing_alone(E, G, keep, top):
    g = torch.Generator().manual_seed(E)
    h = torch.randn(17, 10, generator=g)
    router = torch.randn(E, 10, generator=g)
    want = oracle.route(h.double(), router.double(), top, G, keep, 1.3)
    ex = torch.empty(17, top, dtype=torch.int32)
    wt = torch.empty(17, top)
    ops.route_grouped_topk(ex, wt, h @ router.T, E, G, keep, 1.3)
    for t in range(17):
        a = sorted((int(e), round(float(v), 5)) for e, v in zip(ex[t], wt[t]))
        b = sorted((e, round(v, 5)) for e, v in want[t])
        assert a == b


def test_feed_forward_blocks_alone():
    from gpustack_amd.engine.config import FeedForwardSpec
    from gpustack_amd.models.experts import DenseFF, RoutedFF

    g = torch.Generator().manual_seed(3)
    W = 12
    h = torch.randn(9, W, generator=g)
    d = DenseFF(W, FeedForwardSpec(kind="dense", ff=7, act="relu2"), torch.float32)
    d.up_w.copy_(torch.randn(7, W, generator=g))
    d.down_w.copy_(torch.randn(W, 7, generator=g))
    close(d(h, h), oracle.dense_ff(h.double(), {"up": d.up_w.double(),
                                               "down": d.down_w.double()}), 1e-4)
    for shared in (5, 0):
        f = FeedForwardSpec(kind="moe", ff=4, act="gelu", experts=6, top=3,
                            groups=2, keep_groups=1, route_scale=0.7,
                            shared_ff=shared, shared_gated=bool(shared))
        m = RoutedFF(W, f, torch.float32)
        for p in m.parameters():
            p.copy_(torch.randn(p.shape, generator=g))
        w = {"router": m.router_w[:6].double()}
        for e in range(6):
            w[f"e{e}.up"], w[f"e{e}.down"] = m.up_w[e].double(), m.down_w[e].double()
        if shared:
            w["shared.up"] = m.shared_up_w.double()
            w["shared.down"] = m.shared_down_w.double()
            w["shared.sg"] = m.router_w[6:].double()
        close(m(h, h), oracle.moe_ff(h.double(), w, 6, 3, 2, 1, 0.7,
                                     bool(shared)), 1e-4)


# ---- whole prompts, decoding, portions, batches -----------------------------

def test_whole_prompt_and_every_layer(small):
    cfg, w, d = small
    eng = make_engine(d)
    t = toks(45, cfg["vocab"], 5)
    got = run_schedule(eng, {"a": t}, [[("a", 45)]])["a"]
    close(got, oracle.forward(cfg, w, t))


def test_prefill_against_token_by_token(small):
    cfg, w, d = small
    eng = make_engine(d)
    t = toks(37, cfg["vocab"], 6)
    want = oracle.forward(cfg, w, t)
    whole = run_schedule(eng, {"a": t}, [[("a", 37)]])["a"]
    single = run_schedule(eng, {"b": t}, [[("b", 1)]] * 37)["b"]
    close(whole, want)
    close(single, want)


@pytest.mark.parametrize("cut", [[2, 2, 2, 30, 1, 2, 15, 17, 1, 1, 3, 16, 2],
                                 [15, 1, 16, 1, 17, 44],
                                 [3, 64, 2, 25]])
def test_portions_of_any_size(small, cut):
    cfg, w, d = small
    eng = make_engine(d)
    t = toks(sum(cut), cfg["vocab"], 7)
    got = run_schedule(eng, {"a": t}, [[("a", n)] for n in cut])["a"]
    close(got, oracle.forward(cfg, w, t))


def test_unequal_requests_in_one_batch_equal_each_alone(small):
    cfg, w, d = small
    reqs = {"a": toks(50, cfg["vocab"], 8), "b": toks(3, cfg["vocab"], 9),
            "c": toks(21, cfg["vocab"], 10), "d": toks(1, cfg["vocab"], 11)}
    steps = [[("a", 17), ("b", 2)],
             [("a", 1), ("b", 1), ("c", 16), ("d", 1)],
             [("a", 30), ("c", 1)],
             [("c", 4), ("a", 1)],
             [("a", 1)]]
    got = run_schedule(make_engine(d), reqs, steps)
    for i, t in reqs.items():
        close(got[i], oracle.forward(cfg, w, t))
    alone = {i: run_schedule(make_engine(d), {i: t}, [[(i, len(t))]])[i]
             for i, t in reqs.items()}
    for i in reqs:
        close(got[i], alone[i].double(), 1e-4)


def test_blocks_are_freed_and_used_again(small):
    cfg, w, d = small
    # 6 usable blocks of 16: two 40-token requests cannot both stay
    eng = make_engine(d, blocks=7, max_seqs=2)
    alloc = eng.scheduler.kv.allocator
    free0 = alloc.num_free
    for k in range(4):
        t = toks(40 + k, cfg["vocab"], 20 + k)
        u = toks(30, cfg["vocab"], 40 + k)
        got = run_schedule(eng, {"x": t, "y": u},
                           [[("x", 20), ("y", 30)], [("x", len(t) - 20)]])
        close(got["x"], oracle.forward(cfg, w, t))
        close(got["y"], oracle.forward(cfg, w, u))
        assert alloc.num_free == free0
    with pytest.raises(RuntimeError):
        run_schedule(eng, {"big": toks(200, cfg["vocab"], 1)}, [[("big", 200)]])


def test_first_tokens_of_a_sequence(small):
    cfg, w, d = small
    eng = make_engine(d)
    for seed in range(4):
        t = toks(4, cfg["vocab"], 60 + seed)
        want = oracle.forward(cfg, w, t)
        close(run_schedule(eng, {"a": t}, [[("a", 1)], [("a", 3)]])["a"], want)
        close(run_schedule(eng, {"b": t}, [[("b", 2)], [("b", 2)]])["b"], want)
    # the previous token matters: same token, other predecessor
    a = oracle.forward(cfg, w, [5, 9])[1]
    b = oracle.forward(cfg, w, [6, 9])[1]
    assert (a - b).abs().max() > 1e-3
    got = run_schedule(eng, {"p": [5, 9], "q": [6, 9]},
                       [[("p", 1), ("q", 1)], [("p", 1), ("q", 1)]])
    close(got["p"][1], a)
    close(got["q"][1], b)


def test_long_decoding(small):
    cfg, w, d = small
    eng = make_engine(d)
    t = toks(140, cfg["vocab"], 12)
    got = run_schedule(eng, {"a": t}, [[("a", 10)]] + [[("a", 1)]] * 130)["a"]
    close(got, oracle.forward(cfg, w, t))


def test_bfloat16_engine_stays_near_the_oracle(small):
    cfg, w, d = small
    eng = make_engine(d, dtype="bfloat16")
    t = toks(40, cfg["vocab"], 13)
    got = run_schedule(eng, {"a": t}, [[("a", 23)], [("a", 2)]] + [[("a", 1)]] * 15)["a"]
    want = oracle.forward(cfg, w, t)
    err = (got.double() - want).pow(2).mean().sqrt() / want.pow(2).mean().sqrt()
    assert err < 0.03, err


# ---- other shapes of the design ---------------------------------------------

VARIANTS = {
    "no_pair_table_no_cap": dict(bigram=None, cap=None),
    "one_group": dict(layers=[{"type": "latent_attention", "mixer": mixer(1, 4, 4, 4),
                               "mlp": moe(experts=5, top=5, count=1, keep=1,
                                          shared=0)}]),
    "all_groups_kept": dict(layers=[{"type": "latent_attention",
                                     "mixer": mixer(4, 3, 7, 9, scale=0.9),
                                     "mlp": moe(experts=8, top=3, count=4,
                                                keep=4, ff=3, shared=11)}]),
    "attention_only_layer": dict(layers=[
        {"type": "latent_attention", "mixer": mixer(2, 5, 3, 6), "mlp": None},
        {"type": "latent_attention", "mixer": mixer(5, 2, 2, 3),
         "mlp": {"kind": "dense", "ff": 9}},
        {"type": "latent_attention", "mixer": mixer(1, 16, 1, 20), "mlp": None}]),
    "wide": dict(width=72, vocab=300, bigram=(64, 1, 1), layers=[
        {"type": "latent_attention", "mixer": mixer(7, 16, 24, 40),
         "mlp": moe(experts=12, top=4, count=6, keep=3, ff=32, shared=16)}]),
}


@pytest.mark.parametrize("name", sorted(VARIANTS))
def test_other_configurations(tmp_path, name):
    cfg = make_config(**VARIANTS[name])
    w = make_weights(cfg, seed=len(name))
    eng = make_engine(save_model(tmp_path / "m", cfg, w))
    reqs = {"a": toks(33, cfg["vocab"], 1), "b": toks(18, cfg["vocab"], 2)}
    steps = [[("a", 5), ("b", 16)], [("a", 27), ("b", 1)], [("a", 1), ("b", 1)]]
    got = run_schedule(eng, reqs, steps)
    for i, t in reqs.items():
        close(got[i], oracle.forward(cfg, w, t))


# ---- one key far away decides the output -------------------------------------

def far_key_model(tmp_path, T, targets, R=8):
    """One attention-only layer whose weights make query row r of head a
    match exactly ONE earlier position targets[r][a]: the token table holds
    the wanted stream row per position (token id = position), q reads the
    stream unchanged (W_q = I) and keys are the latents themselves (U_k = I,
    Dq = R), so a query row equal to beta * latent(j) scores beta * |c_j|^2
    on position j and O(beta) elsewhere. If that one key is dropped, read
    from another block or masked one off, the output is another vector."""
    H, Dv = 2, 5
    W = H * R
    cfg = make_config(width=W, vocab=T, bigram=None, cap=None, layers=[
        {"type": "latent_attention", "mixer": mixer(H, R, Dv, R, scale=1.0),
         "mlp": None}])
    w = make_weights(cfg, seed=99)
    w["l0.mix.q"] = torch.eye(W).to(BF)
    w["l0.mix.uk"] = torch.eye(R).repeat(H, 1).to(BF)
    w["l0.mix.dkv.norm"] = torch.ones(R).to(BF)
    g = torch.Generator().manual_seed(7)
    emb = torch.randn(T, W, generator=g).to(BF)
    wd = w["l0.mix.dkv"].double()
    for r, per_head in sorted(targets.items()):
        for a, j in enumerate(per_head):
            assert j < r and j not in targets
            c = oracle.rms_unit(wd @ emb[j].double(), cfg["norm"]["eps"])
            emb[r, a * R:(a + 1) * R] = (6.0 * c).to(BF)
    w["embed"] = emb
    return cfg, w, save_model(tmp_path / "far", cfg, w)


def test_far_keys_and_page_borders(tmp_path):
    T = 200
    # query rows late in the sequence; their keys sit at the first
    # positions, far back, and on both sides of 16-token page borders
    targets = {150: [0, 1], 151: [15, 16], 152: [17, 31], 153: [32, 47],
               160: [48, 63], 175: [64, 127], 176: [128, 143], 177: [144, 149],
               192: [159, 174], 199: [191, 2]}
    cfg, w, d = far_key_model(tmp_path, T, targets)
    t = list(range(T))
    want = oracle.forward(cfg, w, t)
    # the crafted rows really hinge on their one key: hiding it changes them
    hidden = list(t)
    hidden[15] = 3
    assert (oracle.forward(cfg, w, hidden)[151] - want[151]).abs().max() > 0.05
    rows = sorted(targets)
    eng = make_engine(d)
    # in a prompt, whole and in portions that end on / next to the borders
    close(run_schedule(eng, {"a": t}, [[("a", T)]])["a"][rows], want[rows])
    cut = [16, 15, 2, 31, 64, 23, 2, 16, 7, 24]
    close(run_schedule(eng, {"b": t}, [[("b", n)] for n in cut])["b"][rows],
          want[rows])
    # decoded one by one after a prompt that ends inside a page
    steps = [[("c", 149)]] + [[("c", 1)]] * (T - 149)
    close(run_schedule(eng, {"c": t}, steps)["c"][rows], want[rows])


# ---- greedy generation through the engine's own entry point -------------------

def test_greedy_generation(small):
    cfg, w, d = small
    eng = make_engine(d)
    prompts = [toks(9, cfg["vocab"], 30), toks(20, cfg["vocab"], 31), [7]]
    outs = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    for p, o in zip(prompts, outs):
        seq = list(p)
        for _ in range(12):
            seq.append(int(oracle.forward(cfg, w, seq)[-1].argmax()))
        assert o == seq[len(p):]
    # chunked admission of a longer prompt, same answer
    eng2 = make_engine(d)
    eng2.cfg.max_prefill_tokens = 8
    assert eng2.generate([prompts[1]], SamplingParams(
        max_tokens=6, ignore_eos=True))[0] == outs[1][:6]


# ---- the replay command line ---------------------------------------------------

def test_trace_replay_command(small, tmp_path):
    """bin/trace_run: JSON steps on stdin, `done <step>` lines on stdout,
    <step>.f32 files with the wanted logits; a pool of max-tokens is enough
    because ended requests give their blocks back."""
    import subprocess

    import numpy as np

    cfg, w, d = small
    a, b = toks(40, cfg["vocab"], 50), toks(35, cfg["vocab"], 51)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:30], "want": [0, 29]}],
         "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[30:39], "want": []}],
         "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[39:], "want": [0]}],
         "end": ["a"]},
        {"step": 3, "entries": [{"id": "b", "tokens": b, "want": [34, 3]}],
         "end": ["b"]},
    ]
    out = tmp_path / "out"
    exe = Path(__file__).resolve().parent.parent / "bin" / "trace_run"
    r = subprocess.run(
        [sys.executable, str(exe), "--model", d, "--dtype", "float32",
         "--out", str(out), "--max-tokens", "64", "--device", "cpu"],
        input="".join(json.dumps(s) + "\n" for s in steps),
        capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    done = [ln for ln in r.stdout.splitlines() if ln.startswith("done ")]
    assert done == ["done 0", "done 1", "done 2", "done 3"]
    assert not (out / "1.f32").exists()
    wa, wb = oracle.forward(cfg, w, a), oracle.forward(cfg, w, b)
    V = cfg["vocab"]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    close(got0, wa[[0, 29]])
    got2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    close(got2, wa[[39]])
    got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V))
    close(got3, wb[[34, 3]])
