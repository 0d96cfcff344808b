"""Plain float64 oracle of the Fusipel design, written from its equations:
one function per mechanism, whole sequences at once, no cache, no batching,
nothing shared with gpustack_amd. Also the helpers that make small random
configurations and checkpoints for the tests.

Notation: x stream [T, W]; for a mixer H query heads, G kv heads, d the
score size, dv the value size, r = H / G. Linear weights are [out, in].
"""
import json
import math
from pathlib import Path

import torch

F64 = torch.float64
BF = torch.bfloat16


# ---- mechanisms ------------------------------------------------------------

def unit_rms(x, eps, w=None):
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi)
                                       * (z + 0.044715 * z ** 3)))


def rot_freqs(rot):
    """f_i = base^(-2i/dims), i < dims/2; with `scaling`, waves longer than
    original/low are slowed by factor, shorter than original/high kept, and
    blended linearly in between."""
    n = rot["dims"] // 2
    f = [rot["base"] ** (-2.0 * i / rot["dims"]) for i in range(n)]
    sc = rot.get("scaling")
    if sc:
        out = []
        for fi in f:
            wave = 2.0 * math.pi / fi
            if wave < sc["original"] / sc["high"]:
                out.append(fi)
            elif wave > sc["original"] / sc["low"]:
                out.append(fi / sc["factor"])
            else:
                s = (sc["original"] / wave - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1.0 - s) * fi / sc["factor"] + s * fi)
        f = out
    return torch.tensor(f, dtype=F64)


def rotate_pairs(x, rot, pos):
    """x [T, heads, d]: channels (2i, 2i+1), i < dims/2, turn by pos * f_i;
    the angle is formed in 32-bit as the design prescribes."""
    if not rot or not rot.get("dims"):
        return x
    n = rot["dims"] // 2
    ang = (pos.to(torch.float32)[:, None]
           * rot_freqs(rot).to(torch.float32)[None, :]).to(F64)
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    y = x.clone()
    u, v = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
    y[..., 0:2 * n:2] = u * c - v * s
    y[..., 1:2 * n:2] = v * c + u * s
    return y


def visible(T, window=0, keep_first=0):
    """[T, T] bool: row i sees column j."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window:
        ok = ok & ((i - j < window) | (j < keep_first))
    return ok


def softmax_with_sink(s, sink=None):
    """Row softmax of s [T, T] (masked entries -inf); `sink` adds exp(sink)
    to every row's denominator."""
    m = s.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, sink.reshape(1, 1).expand_as(m))
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(sink - m)
    return e / den


def diff_lambda(W, p, diff):
    return (torch.exp((W[p + "lq1"] * W[p + "lk1"]).sum())
            - torch.exp((W[p + "lq2"] * W[p + "lk2"]).sum()) + diff)


def mixer_diff_window(W, p, m, h, eps):
    """Two-map differential attention behind a sliding window that keeps
    the first keys."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, 2 * H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, 2 * G, d)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).view(T, G, dv)
    q = rotate_pairs(q, m.get("rot"), pos)
    k = rotate_pairs(k, m.get("rot"), pos)
    mask = m.get("mask") or {}
    ok = visible(T, mask.get("size", 0), mask.get("keep_first", 0))
    lam = diff_lambda(W, p, m["diff"])
    heads = []
    for a in range(H):
        g = a // (H // G)
        maps = []
        for mp in range(2):
            s = (q[:, 2 * a + mp] @ k[:, 2 * g + mp].T) * m["scale"]
            s = s.masked_fill(~ok, float("-inf"))
            maps.append(softmax_with_sink(s) @ v[:, g])
        o = maps[0] - lam * maps[1]
        heads.append(unit_rms(o, eps) * (1.0 - m["diff"]))
    return torch.cat(heads, -1) @ W[p + "o"].T


def mixer_tied_sink(W, p, m, h, eps):
    """Causal attention whose values are the raw key projections; q and k are
    normed over the whole projection before rotation; per-head sink."""
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(T)
    q = h @ W[p + "q"].T + W[p + "q.b"]
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = k.view(T, G, d)
    q = unit_rms(q, eps, W[p + "q.norm"]).view(T, H, d)
    k = unit_rms(k, eps, W[p + "k.norm"]).view(T, G, d)
    q = rotate_pairs(q, m.get("rot"), pos)
    k = rotate_pairs(k, m.get("rot"), pos)
    ok = visible(T)
    heads = []
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a] @ k[:, g].T) * m["scale"]
        s = s.masked_fill(~ok, float("-inf"))
        heads.append(softmax_with_sink(s, W[p + "sink"][a]) @ v[:, g])
    return torch.cat(heads, -1) @ W[p + "o"].T


def gated_ff(W, p, h):
    return (gelu_tanh(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def layer_order(cfg):
    """[(layer, add the embedding output first)] in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    out = [(i, False) for i in range(lp["start"])]
    for t in range(lp["times"]):
        out += [(i, t > 0 and i == lp["start"])
                for i in range(lp["start"], lp["stop"])]
    return out + [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, weights, tokens, streams=None):
    """Logits [T, vocab] of one whole sequence; `streams` (a list) receives
    the stream after every layer run."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = W["embed"][torch.tensor(tokens)]
    e0 = x.clone()
    for i, inject in layer_order(cfg):
        L, p = cfg["layers"][i], f"l{i}."
        if inject:
            x = x + e0
        fn = mixer_diff_window if L["type"] == "attention" else mixer_tied_sink
        a = fn(W, p + "mix.", L["mixer"], unit_rms(x, eps, W[p + "norm1"]), eps)
        x = x + mult * unit_rms(a, eps, W[p + "norm1b"])
        if L.get("mlp"):
            f = gated_ff(W, p + "mlp.", unit_rms(x, eps, W[p + "norm2"]))
            x = x + mult * unit_rms(f, eps, W[p + "norm2b"])
        if streams is not None:
            streams.append(x.clone())
    return unit_rms(x, eps, W["final.norm"]) @ W["head"].T


def greedy(cfg, weights, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(forward(cfg, weights, toks)[-1].argmax()))
    return toks[len(prompt):]


# ---- small random models ----------------------------------------------------

def rot(dims, base=100.0, scaling=True):
    r = {"dims": dims, "base": base}
    if scaling:
        # wavelengths of a small base straddle both thresholds
        r["scaling"] = {"factor": 3.0, "low": 1.0, "high": 3.0, "original": 40}
    return r


def diff_layer(heads=4, kv_heads=2, dim=6, vdim=10, window=7, keep_first=2,
               diff=0.3, rot_dims=4, ff=24, scale=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": vdim, "diff": diff, "rot": rot(rot_dims),
                      "mask": {"size": window, "keep_first": keep_first},
                      "scale": scale or 1.0 / math.sqrt(dim)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def tied_layer(heads=6, kv_heads=3, dim=8, rot_dims=8, ff=20, scale=None):
    return {"type": "attention_2",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim,
                      "vdim": dim, "rot": rot(rot_dims, base=50.0),
                      "scale": scale or 1.0 / math.sqrt(dim)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(width=20, vocab=61, layers=None, loop=(1, 3, 2), mult=0.7,
                eps=1e-5):
    cfg = {"architecture": "Fusipel", "vocab": vocab, "width": width,
           "norm": {"eps": eps}, "residual_mult": mult,
           "layers": layers if layers is not None else [
               tied_layer(), diff_layer(), tied_layer(heads=2, kv_heads=2,
                                                      dim=10, rot_dims=4),
               diff_layer(heads=3, kv_heads=3, dim=4, vdim=6, window=5,
                          keep_first=0, rot_dims=2, ff=0)]}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0, sink_gain=2.0):
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def lin(o, i, gain=1.0):
        return (torch.randn(o, i, generator=g) * gain / math.sqrt(i)).to(BF)

    def vec(n, base=1.0, spread=0.2):
        return (base + spread * torch.randn(n, generator=g)).to(BF)

    w = {"embed": torch.randn(cfg["vocab"], W, generator=g).to(BF),
         "final.norm": vec(W), "head": lin(cfg["vocab"], W, 2.0)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, d = m["heads"], m["kv_heads"], m["dim"]
        for n in ("norm1", "norm1b"):
            w[p + n] = vec(W)
        if L["type"] == "attention":
            w[p + "mix.q"], w[p + "mix.k"] = lin(2 * H * d, W, 2.0), lin(2 * G * d, W, 2.0)
            w[p + "mix.v"] = lin(G * m["vdim"], W)
            w[p + "mix.q.b"], w[p + "mix.k.b"] = vec(2 * H * d, 0.0, 0.3), vec(2 * G * d, 0.0, 0.3)
            w[p + "mix.v.b"] = vec(G * m["vdim"], 0.0, 0.3)
            for n in ("lq1", "lk1", "lq2", "lk2"):
                w[p + "mix." + n] = vec(d, 0.0, 0.4)
            w[p + "mix.o"] = lin(W, H * m["vdim"])
        else:
            w[p + "mix.q"], w[p + "mix.k"] = lin(H * d, W, 2.0), lin(G * d, W, 2.0)
            w[p + "mix.q.b"], w[p + "mix.k.b"] = vec(H * d, 0.0, 0.3), vec(G * d, 0.0, 0.3)
            w[p + "mix.q.norm"], w[p + "mix.k.norm"] = vec(H * d, 1.5), vec(G * d, 1.5)
            w[p + "mix.sink"] = vec(H, 0.5, sink_gain)
            w[p + "mix.o"] = lin(W, H * d)
        f = L.get("mlp")
        if f:
            for n in ("norm2", "norm2b"):
                w[p + n] = vec(W)
            w[p + "mlp.gate"], w[p + "mlp.up"] = lin(f["ff"], W, 1.5), lin(f["ff"], W)
            w[p + "mlp.down"] = lin(W, f["ff"])
    return w


def save_model(path, cfg, weights):
    from safetensors.torch import save_file

    path = Path(path)
    path.mkdir(parents=True, exist_ok=True)
    (path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in weights.items()},
              str(path / "model.safetensors"))
    return str(path)
