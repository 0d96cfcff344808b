"""Fusipel: a layer-listed decoder on an fp32 stream with a norm before and
after every sublayer and a weight-shared loop over part of the stack.

    x <- x + m * post1(mixer(pre1(x)));   x <- x + m * post2(ff(pre2(x)))

All four are weighted RMS norms and m is one multiplier for the model. The
mixers are two parameterisations of models/paged_attention.py (two-map
differential scores behind a sliding window that keeps the first keys;
whole-projection q/k norm with values tied to the keys and a per-head sink),
the feed-forward is the gated dense block of models/experts.py. The config
may repeat a span of layers several times with the same weights: every pass
has cache pools of its own (ModelSpec.layer_runs / KVCache), and every pass
but the first starts by adding the embedding output to the stream again.

One row kernel (ops.sandwich_add_norm) closes a sublayer and opens the
next: post-norm, multiplier, residual add on the fp32 stream, the optional
embedding re-injection, and the next sublayer's pre-norm in the GEMM dtype.
The model plugs into the engine like the other families (same forward
signature, paged pools from KVCache, the ragged batch view).
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import EngineConfig
from ..parallel import Communicator
from .experts import DenseFF
from .paged_attention import PagedRotaryAttention


class FusipelLayer(nn.Module):
    def __init__(self, width, ls, eps, dtype, comm):
        super().__init__()
        f32 = lambda: nn.Parameter(torch.empty(width, dtype=torch.float32),
                                   requires_grad=False)
        if ls.mixer_type != "paged_attention":
            raise NotImplementedError(ls.mixer_type)
        self.attn = PagedRotaryAttention(width, ls.mixer, eps, dtype, comm)
        self.pre1, self.post1 = f32(), f32()
        if ls.mlp is None:
            self.mlp = None
        else:
            if ls.mlp.kind != "dense":
                raise NotImplementedError(ls.mlp.kind)
            self.mlp = DenseFF(width, ls.mlp, dtype, comm)
            self.pre2, self.post2 = f32(), f32()


class FusipelForCausalLM(nn.Module):
    uses_ragged_meta = True

    def __init__(self, cfg: EngineConfig, comm: Communicator, device):
        super().__init__()
        spec = cfg.spec
        if comm.pp_size > 1 or comm.tp_size > 1:
            raise NotImplementedError(
                "Fusipel serves on one GPU per replica (no TP/PP sharding yet)")
        self.spec, self.cfg, self.comm = spec, cfg, comm
        self.device = torch.device(device)
        dtype = getattr(torch, cfg.dtype)
        self.dtype = dtype
        self.layer_offset = 0
        self.runs = spec.layer_runs()
        self.num_local_layers = len(self.runs)     # cache pools: one per run
        W = spec.hidden_size
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        self.embed = mk(spec.vocab_size, W)
        self.layers = nn.ModuleList(
            [FusipelLayer(W, ls, spec.rms_norm_eps, dtype, comm)
             for ls in spec.layers])
        self.final_norm = mk(W, dt=torch.float32)
        self.lm_head = mk(spec.vocab_size, W)
        self.lm_head_pack = None
        self.offload = None
        self.to(device)

    def post_load(self) -> None:
        for layer in self.layers:
            layer.attn.post_load()

    def graph_capturable(self) -> bool:
        return True

    @torch.inference_mode()
    def forward(self, token_ids, meta, kv, return_hidden: bool = False,
                return_both: bool = False):
        spec = self.spec
        eps, mult = spec.rms_norm_eps, spec.residual_multiplier or 1.0
        T = token_ids.shape[0]
        dev = token_ids.device
        W = spec.hidden_size
        x = torch.empty(T, W, dtype=torch.float32, device=dev)
        h = torch.empty(T, W, dtype=self.dtype, device=dev)
        ops.embed_rows_f32(x, token_ids, self.embed)
        # the embedding output is needed again when a later pass starts
        e0 = x.clone() if any(inj for _, inj in self.runs) else None
        runs = self.runs
        if runs:
            ops.sandwich_add_norm(x, None, None, 0.0, eps, None,
                                  self.layers[runs[0][0]].pre1, h)
        for r, (li, _) in enumerate(runs):
            layer = self.layers[li]
            a = layer.attn(h, meta, kv.k_caches[r], kv.v_caches[r])
            # what the stream meets next: this layer's feed-forward, the
            # next run's mixer (after the re-injection, if it opens a
            # pass), or nothing (the final norm follows on chosen rows)
            if r + 1 < len(runs):
                nxt = self.layers[runs[r + 1][0]].pre1
                inj = e0 if runs[r + 1][1] else None
            else:
                nxt, inj = None, None
            if layer.mlp is not None:
                ops.sandwich_add_norm(x, a, layer.post1, mult, eps, None,
                                      layer.pre2, h)
                f = layer.mlp(h)
                ops.sandwich_add_norm(x, f, layer.post2, mult, eps, inj,
                                      nxt, h)
            else:
                ops.sandwich_add_norm(x, a, layer.post1, mult, eps, inj,
                                      nxt, h)
        rows = x if return_hidden else x[meta.logits_indices]
        y = torch.empty(rows.shape, dtype=self.dtype, device=dev)
        ops.rms_norm_rows(y, rows.contiguous(), self.final_norm, eps)
        if return_hidden:
            return y
        logits = F.linear(y, self.lm_head).float()
        if return_both:
            return logits, y
        return logits
