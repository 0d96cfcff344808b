"""Layer-level comparison bench: a Vunitar stack at real-model layer sizes
beside the closest llama-lineage stack of equal width, depth and heads
(random weights, synthetic tokens). Reports end-to-end prefill and decode
throughput through LLMEngine for both, and per-kernel rates of the new
kernels next to their counterparts with the fraction of the MI355X
roofline each reaches (2.5 PFLOP/s dense bf16, 8 TB/s HBM3E).

Run through `python bench.py --layer-bench [--layer-sizes small,medium]`;
bench.py's default workload is untouched.
"""
from __future__ import annotations

import json
import time

import torch

PEAK_FLOPS = 2.5e15
PEAK_BW = 8.0e12

SIZES = {
    # width, heads, latent width, dense ff, experts, expert ff, layers
    "small": dict(width=1024, heads=8, rank=256, ff=4096, experts=16, eff=512, layers=4),
    "medium": dict(width=2048, heads=16, rank=512, ff=8192, experts=32, eff=1024, layers=4),
    "large": dict(width=4096, heads=32, rank=512, ff=14336, experts=32, eff=2048, layers=2),
}


def vunitar_spec(s, moe: bool):
    from ..engine.config import (FeedForwardSpec, LatentMixerSpec, LayerSpec,
                                 ModelSpec)

    mixer = LatentMixerSpec(heads=s["heads"], qk_dim=128, v_dim=128,
                            kv_rank=s["rank"], scale=128 ** -0.5)
    if moe:
        ff = FeedForwardSpec(kind="moe", ff=s["eff"], act="gelu",
                             experts=s["experts"], top=4, groups=4,
                             keep_groups=2, route_scale=2.0,
                             shared_ff=s["eff"], shared_gated=True)
    else:
        ff = FeedForwardSpec(kind="dense", ff=s["ff"], act="relu2")
    return ModelSpec(
        architecture="Vunitar", vocab_size=32000, hidden_size=s["width"],
        num_layers=s["layers"],
        layers=tuple(LayerSpec("latent_attention", mixer, ff)
                     for _ in range(s["layers"])),
        num_heads=1, num_kv_heads=1, head_dim=8, intermediate_size=0,
        rms_norm_eps=1e-6, max_position_embeddings=1 << 20, eos_token_id=-1,
        norm_after=True, layer_scale=True, fp32_residual=True,
        final_logit_softcap=30.0, bigram_buckets=4093, bigram_mul_prev=131,
        bigram_mul_cur=17)


def llama_spec(s, moe: bool):
    from ..engine.config import ModelSpec

    kw = dict(vocab_size=32000, hidden_size=s["width"],
              intermediate_size=s["ff"], num_layers=s["layers"],
              num_heads=s["heads"], num_kv_heads=max(1, s["heads"] // 4),
              head_dim=128, max_position_embeddings=1 << 20, eos_token_id=-1)
    if moe:
        kw.update(architecture="Qwen3MoeForCausalLM", qk_norm=True,
                  num_experts=s["experts"], num_experts_per_tok=4,
                  moe_intermediate_size=s["eff"])
    return ModelSpec(**kw)


def _engine(spec, device, max_seqs, max_len):
    from ..engine import EngineConfig, LLMEngine

    cfg = EngineConfig(model="layer-bench", device=device, max_num_seqs=max_seqs,
                       max_model_len=max_len, max_prefill_tokens=8192,
                       gpu_memory_utilization=0.5, admission_min_seqs=1)
    cfg.spec = spec
    cfg.max_model_len = max_len
    return LLMEngine(cfg)


def _sync():
    if torch.cuda.is_available():
        torch.cuda.synchronize()


def engine_rates(spec, device, B_pre=8, L=1024, B_dec=64, n_dec=32):
    from ..engine import SamplingParams

    eng = _engine(spec, device, max(B_dec, B_pre), L + n_dec + 8)
    g = torch.Generator().manual_seed(0)
    mk = lambda n: torch.randint(2, spec.vocab_size, (n,), generator=g).tolist()

    def prefill_once():
        for _ in range(B_pre):
            eng.add_request(mk(L), SamplingParams(max_tokens=1, ignore_eos=True))
        while eng.has_unfinished():
            eng.step()

    prefill_once()
    _sync()
    t0 = time.perf_counter()
    reps = 3
    for _ in range(reps):
        prefill_once()
    _sync()
    pre = reps * B_pre * L / (time.perf_counter() - t0)

    for _ in range(B_dec):
        eng.add_request(mk(L), SamplingParams(max_tokens=n_dec + 8,
                                              ignore_eos=True))
    while eng.num_running < B_dec and eng.has_unfinished():
        eng.step()
    for _ in range(4):
        eng.step()
    _sync()
    t0 = time.perf_counter()
    steps = n_dec - 8
    for _ in range(steps):
        eng.step()
    _sync()
    dec = steps * B_dec / (time.perf_counter() - t0)
    while eng.has_unfinished():
        eng.step()
    del eng
    if torch.cuda.is_available():
        torch.cuda.empty_cache()
    return pre, dec


def _time(fn, iters=20):
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(True), torch.cuda.Event(True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters * 1e-3


def kernel_rates(s, device):
    """Per-kernel rates: (name, seconds, achieved, unit, roofline share)."""
    from .. import ops

    bf = torch.bfloat16
    H, R, W, D, BS = s["heads"], s["rank"], s["width"], 128, 16
    out = []

    def rec(name, sec, flops=None, nbytes=None):
        if flops is not None:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            tflops=round(flops / sec / 1e12, 1),
                            roofline=round(flops / sec / PEAK_FLOPS, 4)))
        else:
            out.append(dict(kernel=name, us=round(sec * 1e6, 1),
                            gbps=round(nbytes / sec / 1e9, 1),
                            roofline=round(nbytes / sec / PEAK_BW, 4)))

    # ---- prefill attention: 4 prompts x 2048 ----
    nseq, L = 4, 2048
    T = nseq * L
    pairs = nseq * L * (L + 1) // 2
    nblk = T // BS + 1
    pool = torch.randn(nblk, 2, BS, R, device=device).to(bf)
    bt = torch.arange(nseq * (L // BS), dtype=torch.int32, device=device).view(nseq, -1)
    row_seq = torch.arange(nseq, dtype=torch.int32, device=device).repeat_interleave(L)
    pos = torch.arange(L, dtype=torch.int32, device=device).repeat(nseq)
    q = torch.randn(T, H, R, device=device) * R ** -0.5
    ctx = torch.empty_like(q)
    tiles = ops.build_latent_tiles([i * L for i in range(nseq)], [0] * nseq,
                                   [L] * nseq, H, device)
    rec("latent_attention prefill (mfma)",
        _time(lambda: ops.latent_attention(ctx, q, pool, bt, row_seq, pos, 1.0,
                                           tiles=tiles), 5),
        flops=4.0 * R * H * pairs)
    qf = torch.randn(T, H, D, device=device).to(bf)
    kf = torch.randn(T, max(1, H // 4), D, device=device).to(bf)
    vf = torch.randn_like(kf)
    of = torch.empty_like(qf)
    ptiles = ops.build_prefill_tiles([L] * nseq, device)
    rec("flash_prefill (llama graph)",
        _time(lambda: ops.varlen_prefill_attn(of, qf, kf, vf, [L] * nseq,
                                              D ** -0.5, tiles=ptiles), 5),
        flops=4.0 * D * H * pairs)

    # ---- decode attention: 64 sequences x 2048 cached ----
    B, Lc = 64, 2048
    nblk = B * (Lc // BS) + 1
    pool = torch.randn(nblk, 2, BS, R, device=device).to(bf)
    bt = torch.arange(B * (Lc // BS), dtype=torch.int32, device=device).view(B, -1)
    row_seq = torch.arange(B, dtype=torch.int32, device=device)
    pos = torch.full((B,), Lc - 1, dtype=torch.int32, device=device)
    q = torch.randn(B, H, R, device=device) * R ** -0.5
    ctx = torch.empty_like(q)
    tiles = ops.build_latent_tiles(list(range(B)), [Lc - 1] * B, [1] * B, H, device)
    rec("latent_attention decode (mfma)",
        _time(lambda: ops.latent_attention(ctx, q, pool, bt, row_seq, pos, 1.0,
                                           tiles=tiles, max_ctx=Lc)),
        nbytes=B * Lc * R * 2 * 2)
    hkv = max(1, H // 4)
    kc = torch.randn(nblk, hkv, BS, D, device=device).to(bf)
    vc = torch.randn_like(kc)
    qd = torch.randn(B, H, D, device=device).to(bf)
    od = torch.empty_like(qd)
    lens = torch.full((B,), Lc, dtype=torch.int32, device=device)
    rec("paged_attn_decode (llama graph)",
        _time(lambda: ops.paged_attn_decode(od, qd, kc, vc, bt, lens, D ** -0.5)),
        nbytes=B * Lc * hkv * D * 2 * 2)

    # ---- row kernels at T = 8192 ----
    T = 8192
    x = torch.randn(T, W, device=device)
    a = torch.randn(T, W, device=device).to(bf)
    w32 = torch.ones(W, device=device)
    hb = torch.empty(T, W, dtype=bf, device=device)
    rec("rms_scale_add (fp32 stream + bf16 copy)",
        _time(lambda: ops.rms_scale_add(x, a, w32, w32, 1e-6, hb)),
        nbytes=T * W * 12)
    xb, rb = a.clone(), a.clone()
    wb = torch.ones(W, dtype=bf, device=device)
    rec("fused_add_rms_norm (llama graph)",
        _time(lambda: ops.fused_add_rms_norm(xb, rb, wb, 1e-6)),
        nbytes=T * W * 8)
    u = torch.randn(T, s["ff"], device=device).to(bf)
    rec("act_inplace relu2", _time(lambda: ops.act_inplace(u, "relu2")),
        nbytes=T * s["ff"] * 4)
    gu = torch.randn(T, 2 * s["ff"], device=device).to(bf)
    ao = torch.empty(T, s["ff"], dtype=bf, device=device)
    rec("silu_and_mul (llama graph)", _time(lambda: ops.silu_and_mul(ao, gu)),
        nbytes=T * s["ff"] * 6)
    nblk = T // BS + 1
    pool = torch.zeros(nblk, 2, BS, R, dtype=bf, device=device)
    src = torch.randn(T, H * D + R, device=device).to(bf)
    slots = torch.arange(T, device=device)      # a prompt: consecutive slots
    rec("latent_norm_store (norm + both planes)",
        _time(lambda: ops.latent_norm_store(pool, src, H * D, w32[:R].contiguous()
                                            if R <= W else torch.ones(R, device=device),
                                            slots, 1e-6)),
        nbytes=T * R * 6)
    hkv = max(1, H // 4)
    kk = torch.randn(T, hkv, D, device=device).to(bf)
    kc = torch.zeros(nblk, hkv, BS, D, dtype=bf, device=device)
    vc = torch.zeros_like(kc)
    rec("reshape_and_cache (llama graph)",
        _time(lambda: ops.reshape_and_cache(kk, kk, kc, vc, slots)),
        nbytes=T * hkv * D * 8)
    return out


def run(sizes: list[str], device: str) -> None:
    for name in sizes:
        s = SIZES[name]
        for moe in (False, True):
            row = {"size": name, **s, "ff_kind": "moe" if moe else "dense"}
            for label, mk in (("vunitar", vunitar_spec), ("llama_graph", llama_spec)):
                pre, dec = engine_rates(mk(s, moe), device)
                row[label] = {"prefill_tok_s": round(pre), "decode_tok_s": round(dec)}
            print(json.dumps({"layer_bench": row}), flush=True)
        if torch.cuda.is_available():
            for k in kernel_rates(s, device):
                print(json.dumps({"kernel_bench": {"size": name, **k}}), flush=True)
