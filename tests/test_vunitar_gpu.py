"""Vunitar on the GPU: the engine with the HIP kernels (fp32 exact path,
bf16 MFMA attention, grouped expert kernels, captured decode graphs)
against the float64 oracle, on the schedules of tests/test_vunitar.py."""
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import test_vunitar as tv  # noqa: E402
import vunitar_oracle as oracle  # noqa: E402

from gpustack_amd import ops  # noqa: E402
from gpustack_amd.engine import SamplingParams  # noqa: E402

pytestmark = pytest.mark.gpu

# sizes the MFMA attention (latent width % 32) and the grouped expert
# kernels (width, ff % 64) accept, still unlike each other
ALIGNED = dict(width=64, vocab=97, bigram=(29, 3, 5), layers=[
    {"type": "latent_attention", "mixer": tv.mixer(3, 16, 24, 32),
     "mlp": {"kind": "dense", "ff": 80}},
    {"type": "latent_attention", "mixer": tv.mixer(2, 8, 8, 96),
     "mlp": tv.moe(experts=8, top=3, count=2, keep=1, ff=64, shared=48)},
    {"type": "latent_attention", "mixer": tv.mixer(5, 8, 16, 64), "mlp": None},
])

REQS = {"a": 50, "b": 3, "c": 21, "d": 1}
STEPS = [[("a", 17), ("b", 2)], [("a", 1), ("b", 1), ("c", 16), ("d", 1)],
         [("a", 30), ("c", 1)], [("c", 4), ("a", 1)], [("a", 1)]]


@pytest.fixture
def gpu_engine():
    """Engine factory whose engines are torn down when the test is over:
    an engine is a reference cycle (runner <-> graph runner), so without an
    explicit collection its captured graphs and pool would linger into
    whatever runs next in the process."""
    import gc

    made = []

    def make(model_dir, **kw):
        made.append(tv.make_engine(model_dir, device="cuda", **kw))
        return made[-1]

    yield make
    made.clear()
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def _model(tmp_path, kw, seed=3):
    cfg = tv.make_config(**kw)
    w = tv.make_weights(cfg, seed=seed)
    return cfg, w, tv.save_model(tmp_path / "m", cfg, w)


@pytest.mark.parametrize("name", ["default", "wide", "aligned"])
def test_fp32_engine_matches_oracle(tmp_path, gpu_engine, name):
    kw = {"default": {}, "wide": tv.VARIANTS["wide"], "aligned": ALIGNED}[name]
    cfg, w, d = _model(tmp_path, kw)
    eng = gpu_engine(d)
    reqs = {i: tv.toks(n, cfg["vocab"], 70 + n) for i, n in REQS.items()}
    got = tv.run_schedule(eng, reqs, STEPS)
    for i, t in reqs.items():
        tv.close(got[i], oracle.forward(cfg, w, t), 2e-3)


def test_bf16_engine_mfma_and_grouped_experts(tmp_path, gpu_engine):
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16", blocks=12)
    assert ops._load_latent().latent_attention_uses_mfma(eng.runner.kv.k_caches[0])
    for rnd in range(3):      # blocks are freed and taken again
        reqs = {i: tv.toks(n, cfg["vocab"], 80 + n + rnd) for i, n in REQS.items()}
        got = tv.run_schedule(eng, reqs, STEPS)
        for i, t in reqs.items():
            want = oracle.forward(cfg, w, t)
            err = ((got[i].double() - want).pow(2).mean().sqrt()
                   / want.pow(2).mean().sqrt())
            assert err < 0.03, (i, float(err))


@pytest.mark.parametrize("dtype,R", [("float32", 8), ("bfloat16", 8),
                                     ("bfloat16", 32)])
def test_far_keys_and_page_borders(tmp_path, gpu_engine, dtype, R):
    T = 200
    targets = {150: [0, 1], 151: [15, 16], 152: [17, 31], 153: [32, 47],
               160: [48, 63], 175: [64, 127], 176: [128, 143], 177: [144, 149],
               192: [159, 174], 199: [191, 2]}
    cfg, w, d = tv.far_key_model(tmp_path, T, targets, R=R)
    t = list(range(T))
    want = oracle.forward(cfg, w, t)
    rows = sorted(targets)
    eng = gpu_engine(d, dtype=dtype)
    tol = 2e-3 if dtype == "float32" else 0.15
    tv.close(tv.run_schedule(eng, {"a": t}, [[("a", T)]])["a"][rows], want[rows], tol)
    cut = [16, 15, 2, 31, 64, 23, 2, 16, 7, 24]
    tv.close(tv.run_schedule(eng, {"b": t}, [[("b", n)] for n in cut])["b"][rows],
             want[rows], tol)
    steps = [[("c", 149)]] + [[("c", 1)]] * (T - 149)
    tv.close(tv.run_schedule(eng, {"c": t}, steps)["c"][rows], want[rows], tol)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_generation_agrees_with_replay(tmp_path, gpu_engine, dtype):
    """Greedy generation (scheduler, decode batches; captured graphs for the
    bf16 engine) must pick the tokens that the forced-token path scores
    highest at the same places."""
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype=dtype, blocks=64, max_seqs=8)
    if dtype == "bfloat16":
        assert eng.runner.graph_runner is not None
    prompts = [tv.toks(n, cfg["vocab"], 90 + n) for n in (9, 20, 1, 33)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=24, ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert len(o) == 24
        full = p + o
        lg = tv.run_schedule(eng, {"r": full}, [[("r", len(full))]])["r"]
        for k, tok in enumerate(o):
            row = lg[len(p) + k - 1]
            top2 = row.topk(2).values
            if top2[0] - top2[1] > 0.05:      # skip near-ties
                assert int(row.argmax()) == tok, (k, tok)


@pytest.mark.parametrize("E,W,F,T,top", [(8, 64, 64, 5, 3), (4, 128, 192, 40, 2),
                                         (16, 576, 128, 17, 4)])
def test_grouped_expert_kernels(E, W, F, T, top):
    g = torch.Generator().manual_seed(E + T)
    bf = torch.bfloat16
    x = torch.randn(T, W, generator=g).to(bf).cuda()
    up = (torch.randn(E, F, W, generator=g) / W ** 0.5).to(bf).cuda()
    down = (torch.randn(E, W, F, generator=g) / F ** 0.5).to(bf).cuda()
    ex = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)])
    ex[:, 0] = 1                    # one crowded expert, several empty ones
    flat = ex.reshape(-1).cuda()
    order = torch.argsort(flat, stable=True)
    counts = torch.bincount(flat, minlength=E).to(torch.int32)
    offs = (counts.cumsum(0) - counts).to(torch.int32)
    s_tok = (order // top).to(torch.int32)
    u = torch.empty(T * top, F, dtype=bf, device="cuda")
    y = torch.empty(T * top, W, dtype=bf, device="cuda")
    ops.grouped_up_act(u, x, up, s_tok, offs, counts, "gelu")
    ops.grouped_down(y, u, down, offs, counts)
    xs = x[s_tok.long()].float()
    e_of = flat[order]
    ru = torch.nn.functional.gelu(torch.einsum("jw,jfw->jf", xs, up.float()[e_of]))
    torch.testing.assert_close(u.float(), ru, rtol=2e-2, atol=2e-2)
    ry = torch.einsum("jf,jwf->jw", u.float(), down.float()[e_of])
    torch.testing.assert_close(y.float(), ry, rtol=2e-2, atol=2e-2)
