"""Plain, slow Vunitar forward pass used as the test oracle.

One function per mechanism, written straight from the design's equations
in float64 torch on the CPU. It shares no code with the serving path: no
paged cache, no batching, no kernels — every call recomputes the whole
sequence from position 0.

Notation: W = residual width, H = heads, Dq = query/key dims per head,
Dv = value dims per head, R = latent width, E = experts, G = expert groups.
Weights arrive as a dict name -> tensor with the checkpoint's own names.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def embed_tokens(tokens: list[int], embed: torch.Tensor,
                 bigram: torch.Tensor | None, buckets: int, mul_prev: int,
                 mul_cur: int) -> torch.Tensor:
    """Token row plus a hashed (previous, current) pair row; the first
    token of a sequence takes the table's extra last row."""
    rows = []
    for i, t in enumerate(tokens):
        x = embed[t].clone()
        if bigram is not None:
            r = buckets if i == 0 else (tokens[i - 1] * mul_prev
                                        + t * mul_cur) % buckets
            x = x + bigram[r]
        rows.append(x)
    return torch.stack(rows)


def latent_attention(h: torch.Tensor, w: dict, heads: int, dq: int, dv: int,
                     rank: int, scale: float, eps: float) -> torch.Tensor:
    """Causal softmax attention whose keys and values are both linear
    images of one normalised low-rank latent per token; no positional
    signal enters the scores."""
    T = h.shape[0]
    q = (h @ w["q"].T).view(T, heads, dq)
    c = rms_norm(h @ w["dkv"].T, w["dkv.norm"], eps)          # [T, R]
    k = (c @ w["uk"].T).view(T, heads, dq)
    v = (c @ w["uv"].T).view(T, heads, dv)
    out = torch.zeros(T, heads, dv, dtype=h.dtype)
    for i in range(T):
        for a in range(heads):
            s = (k[: i + 1, a] @ q[i, a]) * scale            # [i+1]
            p = torch.softmax(s, dim=0)
            out[i, a] = p @ v[: i + 1, a]
    return out.reshape(T, heads * dv) @ w["o"].T


def relu_squared(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z) ** 2


def gelu_erf(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))


def dense_ff(h: torch.Tensor, w: dict) -> torch.Tensor:
    return relu_squared(h @ w["up"].T) @ w["down"].T


def route(h: torch.Tensor, router: torch.Tensor, top: int, groups: int,
          keep: int, scale: float):
    """Softmax over all experts; whole groups of neighbouring experts are
    ranked by their best member and only the `keep` best groups stay
    eligible; the `top` best eligible experts are taken with weight
    score * scale (no renormalisation). Returns per token a list of
    (expert, weight)."""
    s = torch.softmax(h @ router.T, dim=-1)                  # [T, E]
    T, E = s.shape
    per = E // groups
    picks = []
    for t in range(T):
        gbest = [max(float(s[t, g * per + j]) for j in range(per))
                 for g in range(groups)]
        order = sorted(range(groups), key=lambda g: -gbest[g])[:keep]
        allowed = [g * per + j for g in order for j in range(per)]
        allowed.sort(key=lambda e: -float(s[t, e]))
        picks.append([(e, float(s[t, e]) * scale) for e in allowed[:top]])
    return picks


def moe_ff(h: torch.Tensor, w: dict, experts: int, top: int, groups: int,
           keep: int, scale: float, shared: bool) -> torch.Tensor:
    picks = route(h, w["router"], top, groups, keep, scale)
    out = torch.zeros_like(h)
    for t, chosen in enumerate(picks):
        for e, wt in chosen:
            y = gelu_erf(h[t] @ w[f"e{e}.up"].T) @ w[f"e{e}.down"].T
            out[t] += wt * y
    if shared:
        y = gelu_erf(h @ w["shared.up"].T) @ w["shared.down"].T
        gate = torch.sigmoid(h @ w["shared.sg"].T)           # [T, 1]
        out = out + gate * y
    return out


def _sub(weights: dict, prefix: str) -> dict:
    n = len(prefix)
    return {k[n:]: v for k, v in weights.items() if k.startswith(prefix)}


def forward(cfg: dict, weights: dict, tokens: list[int],
            collect_layers: bool = False):
    """Logits [T, vocab] for one sequence; optionally also the residual
    stream after every layer."""
    wt = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    bg = (cfg.get("embedding") or {}).get("bigram")
    x = embed_tokens(tokens, wt["embed"], wt.get("bigram") if bg else None,
                     bg["buckets"] if bg else 0,
                     bg["mul_prev"] if bg else 0, bg["mul_cur"] if bg else 0)
    per_layer = []
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        if L["type"] != "latent_attention":
            raise ValueError(L["type"])
        m = L["mixer"]
        a = latent_attention(x, _sub(wt, p + "mix."), m["heads"], m["dim"],
                             m["vdim"], m["kv_rank"], m["scale"], eps)
        x = x + rms_norm(a, wt[p + "norm1"], eps) * wt[p + "ls1"]
        mlp = L.get("mlp")
        if mlp:
            mw = _sub(wt, p + "mlp.")
            if mlp["kind"] == "dense":
                f = dense_ff(x, mw)
            else:
                r = mlp["router"]
                f = moe_ff(x, mw, r["experts"], r["top"],
                           r["groups"]["count"], r["groups"]["keep"],
                           r["scale"], bool(mlp.get("shared")))
            x = x + rms_norm(f, wt[p + "norm2"], eps) * wt[p + "ls2"]
        per_layer.append(x.clone())
    y = rms_norm(x, wt["final.norm"], eps)
    logits = y @ wt["head"].T
    cap = cfg.get("logit_softcap")
    if cap:
        logits = cap * torch.tanh(logits / cap)
    if collect_layers:
        return logits, torch.stack(per_layer)
    return logits
