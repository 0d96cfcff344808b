"""Fusipel on the GPU: the engine with the HIP kernels (fp32 vector-ALU
attention, bf16 MFMA attention with key split, fused row kernels, captured
decode graphs) against the float64 oracle, on the schedules and the crafted
cases of tests/test_fusipel.py."""
import sys
from pathlib import Path

import pytest
import torch

sys.path.insert(0, str(Path(__file__).resolve().parent))
import fusipel_oracle as oracle  # noqa: E402
import test_fusipel as tf  # noqa: E402

from gpustack_amd import ops  # noqa: E402
from gpustack_amd.engine import SamplingParams  # noqa: E402

pytestmark = pytest.mark.gpu

# sizes the MFMA attention accepts (score size % 32, value size % 16), still
# unlike each other and unlike the kv grouping of the small default model
ALIGNED = dict(width=64, vocab=97, loop=(0, 2, 2), layers=[
    oracle.tied_layer(heads=4, kv_heads=2, dim=32, rot_dims=8, ff=80),
    oracle.diff_layer(heads=6, kv_heads=3, dim=32, vdim=48, window=37,
                      keep_first=5, rot_dims=16, ff=0),
    oracle.tied_layer(heads=2, kv_heads=2, dim=64, rot_dims=64, ff=48),
    oracle.diff_layer(heads=3, kv_heads=1, dim=64, vdim=16, window=20,
                      keep_first=0, rot_dims=4, ff=32),
])

REQS = {"a": 150, "b": 3, "c": 61, "d": 1}
STEPS = [[("a", 47), ("b", 2)], [("a", 1), ("b", 1), ("c", 16), ("d", 1)],
         [("a", 90), ("c", 1)], [("c", 43), ("a", 1)], [("a", 11), ("c", 1)]]


@pytest.fixture
def gpu_engine():
    """Engine factory whose engines are torn down when the test is over:
    an engine is a reference cycle (runner <-> graph runner), so without an
    explicit collection its captured graphs and pool would linger into
    whatever runs next in the process."""
    import gc

    made = []

    def make(model_dir, **kw):
        made.append(tf.make_engine(model_dir, device="cuda", **kw))
        return made[-1]

    yield make
    made.clear()
    gc.collect()
    torch.cuda.synchronize()
    torch.cuda.empty_cache()


def _model(tmp_path, kw, seed=3):
    cfg = oracle.make_config(**kw)
    w = oracle.make_weights(cfg, seed=seed)
    return cfg, w, oracle.save_model(tmp_path / "m", cfg, w)


@pytest.mark.parametrize("name", ["default", "aligned"])
def test_fp32_engine_matches_oracle(tmp_path, gpu_engine, name):
    cfg, w, d = _model(tmp_path, {} if name == "default" else ALIGNED)
    eng = gpu_engine(d)
    reqs = {i: tf.tokens_for(cfg, n, 70 + n) for i, n in REQS.items()}
    got = tf.replay(eng, reqs, STEPS)
    for i, t in reqs.items():
        assert tf.err(got[i], oracle.forward(cfg, w, t)) < 5e-4, i


@pytest.mark.parametrize("name", ["default", "aligned"])
def test_bf16_engine_and_block_reuse(tmp_path, gpu_engine, name):
    """bf16 serving path (MFMA attention for the aligned sizes, the fp32
    vector path for the others) in a pool that every repetition refills."""
    cfg, w, d = _model(tmp_path, {} if name == "default" else ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16", blocks=18)
    if name == "aligned":
        kv = eng.runner.kv
        q = torch.empty(1, 4, 32, dtype=torch.bfloat16, device="cuda")
        assert ops._load_paged().paged_attention_uses_mfma(
            q, kv.k_caches[0], kv.v_caches[0])
    for rnd in range(3):
        reqs = {i: tf.tokens_for(cfg, n, 80 + n + rnd) for i, n in REQS.items()}
        got = tf.replay(eng, reqs, STEPS)
        for i, t in reqs.items():
            assert tf.err(got[i], oracle.forward(cfg, w, t)) < 0.15, (rnd, i)


def test_bf16_logits_do_not_depend_on_the_schedule(tmp_path, gpu_engine):
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16")
    reqs = {i: tf.tokens_for(cfg, n, 90 + n) for i, n in REQS.items()}
    mixed = tf.replay(eng, reqs, STEPS)
    for i, t in reqs.items():
        whole = tf.replay(eng, {i: t}, [[(i, len(t))]])[i]
        ref = oracle.forward(cfg, w, t)
        # both are rounding away from the oracle, and no further from each
        # other than from it
        assert tf.err(mixed[i], whole.double()) < 0.15, i
        assert tf.err(whole, ref) < 0.15, i


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.12)])
@pytest.mark.parametrize("far_pos", [0, 16, 63, 64, 500])
def test_far_key_among_hundreds(tmp_path, gpu_engine, dtype, tol, far_pos):
    """One key stands out among 1100 (tests/test_fusipel.py standout_model);
    as the last row of a prompt and as a decoded token, where the MFMA
    kernel splits the keys over workgroups."""
    cfg, w, d, toks = tf.standout_model(tmp_path, far_pos, 1100)
    ref = oracle.forward(cfg, w, toks)[-1:]
    eng = gpu_engine(d, dtype=dtype, blocks=80)
    n = len(toks)
    a = tf.replay(eng, {"a": toks}, [[("a", n)]])["a"][-1:]
    b = tf.replay(eng, {"a": toks}, [[("a", n - 1)], [("a", 1)]])["a"][-1:]
    assert tf.err(a, ref) < tol and tf.err(b, ref) < tol


@pytest.mark.parametrize("dtype,tol", [("float32", 5e-4), ("bfloat16", 0.12)])
@pytest.mark.parametrize("gap", [0, 1])
@pytest.mark.parametrize("edge", ["window", "first"])
def test_window_and_kept_keys_edges(tmp_path, gpu_engine, dtype, tol, gap, edge):
    n, window, keep = 211, 70, 18       # edges inside pages and key tiles
    far_pos = (n - 1) - (window - 1) - gap if edge == "window" else keep - 1 + gap
    cfg, w, d, toks = tf.standout_model(tmp_path, far_pos, n, window, keep,
                                        kind="diff")
    ref = oracle.forward(cfg, w, toks)[-1:]
    eng = gpu_engine(d, dtype=dtype)
    a = tf.replay(eng, {"a": toks}, [[("a", 100)], [("a", n - 100)]])["a"][-1:]
    b = tf.replay(eng, {"a": toks}, [[("a", n - 1)], [("a", 1)]])["a"][-1:]
    assert tf.err(a, ref) < tol and tf.err(b, ref) < tol


def test_generation_with_decode_graphs(tmp_path, gpu_engine):
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d)
    assert eng.runner.graph_runner is not None
    prompts = [tf.tokens_for(cfg, n, 40 + n) for n in (3, 70, 9)]
    outs = eng.generate(prompts, SamplingParams(max_tokens=40, temperature=0.0,
                                                ignore_eos=True))
    for p, o in zip(prompts, outs):
        assert o == oracle.greedy(cfg, w, p, 40)


def test_bf16_generation_runs_and_stays_close(tmp_path, gpu_engine):
    """bf16 greedy decoding may part from the oracle at a near-tie; the
    logits of the tokens it did choose must still be the oracle's."""
    cfg, w, d = _model(tmp_path, ALIGNED)
    eng = gpu_engine(d, dtype="bfloat16")
    prompt = tf.tokens_for(cfg, 30, 5)
    out = eng.generate([prompt], SamplingParams(max_tokens=24, temperature=0.0,
                                                ignore_eos=True))[0]
    assert len(out) == 24
    full = prompt + out
    got = tf.replay(eng, {"z": full}, [[("z", len(full))]])["z"]
    assert tf.err(got, oracle.forward(cfg, w, full)) < 0.15
