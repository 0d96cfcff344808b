"""Vunitar: a decoder whose config lists its layers one by one.

Each layer names its mixer (latent attention, models/latent_attention.py)
and feed-forward (dense or routed, models/experts.py; or none) with their
own sizes. The layer flow is norm-after with layer scale on an fp32 stream:

    x <- x + s1 * rmsnorm1(mixer(x));   x <- x + s2 * rmsnorm2(ff(x))

Token rows get a hashed (previous token, token) pair embedding added; the
final logits pass a tanh soft cap. The model plugs into the engine like
LlamaForCausalLM (same forward signature, paged pool from KVCache, batches
from the scheduler) and asks the runner for the ragged batch view
(`uses_ragged_meta`), which also carries each row's previous token.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import EngineConfig
from ..parallel import Communicator
from .experts import DenseFF, RoutedFF
from .latent_attention import LatentAttention


class VunitarLayer(nn.Module):
    def __init__(self, width, ls, eps, dtype, comm):
        super().__init__()
        self.eps = eps
        f32 = lambda: nn.Parameter(torch.empty(width, dtype=torch.float32),
                                   requires_grad=False)
        if ls.mixer_type != "latent_attention":
            raise NotImplementedError(ls.mixer_type)
        self.attn = LatentAttention(width, ls.mixer, eps, dtype, comm)
        self.norm1, self.ls1 = f32(), f32()
        if ls.mlp is None:
            self.mlp = None
        else:
            cls = RoutedFF if ls.mlp.kind == "moe" else DenseFF
            self.mlp = cls(width, ls.mlp, dtype, comm)
            self.norm2, self.ls2 = f32(), f32()

    def forward(self, x, h, meta, cache):
        """x: fp32 stream (updated in place); h: x in the GEMM dtype (x
        itself when the engine runs fp32)."""
        h_out = None if h is x else h
        a = self.attn(h, meta, cache)
        ops.rms_scale_add(x, a, self.norm1, self.ls1, self.eps, h_out)
        if self.mlp is not None:
            f = self.mlp(h, x)
            ops.rms_scale_add(x, f, self.norm2, self.ls2, self.eps, h_out)


class VunitarForCausalLM(nn.Module):
    uses_ragged_meta = True

    def __init__(self, cfg: EngineConfig, comm: Communicator, device):
        super().__init__()
        spec = cfg.spec
        if comm.pp_size > 1 or comm.tp_size > 1:
            raise NotImplementedError(
                "Vunitar serves on one GPU per replica (no TP/PP sharding yet)")
        self.spec, self.cfg, self.comm = spec, cfg, comm
        self.device = torch.device(device)
        dtype = getattr(torch, cfg.dtype)
        self.dtype = dtype
        self.layer_offset = 0
        self.num_local_layers = spec.num_layers
        W = spec.hidden_size
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        self.embed = mk(spec.vocab_size, W)
        self.pair_table = (mk(spec.bigram_buckets + 1, W)
                           if spec.bigram_buckets else None)
        self.layers = nn.ModuleList(
            [VunitarLayer(W, ls, spec.rms_norm_eps, dtype, comm)
             for ls in spec.layers])
        self.final_norm = mk(W, dt=torch.float32)
        self.lm_head = mk(spec.vocab_size, W)
        self.lm_head_pack = None
        self.offload = None
        self.to(device)

    def graph_capturable(self) -> bool:
        """True when a decode step runs without any host sync, so the
        runner may capture it into a hipGraph: every routed feed-forward
        must be able to take the grouped (sync-free) expert kernels."""
        import os

        for layer in self.layers:
            m = layer.mlp
            if isinstance(m, RoutedFF) and not (
                    self.dtype == torch.bfloat16
                    and self.spec.hidden_size % 64 == 0 and m.f.ff % 64 == 0
                    and os.environ.get("GPUSTACK_AMD_FUSED_MOE", "1") == "1"):
                return False
        return True

    @torch.inference_mode()
    def forward(self, token_ids, meta, kv, return_hidden: bool = False,
                return_both: bool = False):
        spec = self.spec
        rg = meta.ragged
        T = token_ids.shape[0]
        dev = token_ids.device
        x = torch.empty(T, spec.hidden_size, dtype=torch.float32, device=dev)
        h = x if self.dtype == torch.float32 else torch.empty(
            T, spec.hidden_size, dtype=self.dtype, device=dev)
        ops.embed_pair_hash(x, None if h is x else h, token_ids,
                            rg.prev_tokens, self.embed, self.pair_table,
                            spec.bigram_buckets, spec.bigram_mul_prev,
                            spec.bigram_mul_cur)
        for i, layer in enumerate(self.layers):
            layer(x, h, meta, kv.k_caches[i])
        rows = x if return_hidden else x[meta.logits_indices]
        y = torch.empty(rows.shape, dtype=self.dtype, device=dev)
        ops.rms_norm_f32(y, rows, self.final_norm, spec.rms_norm_eps)
        if return_hidden:
            return y
        logits = F.linear(y, self.lm_head).float()
        if spec.final_logit_softcap:
            ops.softcap_(logits, spec.final_logit_softcap)
        if return_both:
            return logits, y
        return logits
