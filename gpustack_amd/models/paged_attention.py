"""Rotary softmax attention over a paged key/value pool, for models on the
fp32 stream (ModelSpec.fp32_residual). One module covers a family of
variants, every one a parameter of PagedMixerSpec:

* grouped-query heads with own key and value widths, projection biases;
* pairwise rotary on the first channels of each head, with optional
  wavelength-dependent frequency scaling; angles are pos * f in fp32;
* weighted RMS norm over the whole q / k projection before rotation;
* values tied to the keys (the raw key projection: not normed, not rotated);
* a sliding window that also keeps the first keys of the sequence;
* a per-head sink logit in the softmax denominator;
* differential scores: two score maps per head share one value stream,
  out = unit_rms(a1 - lambda * a2) * (1 - diff), lambda = exp(lq1.lk1) -
  exp(lq2.lk2) + diff.

Flow per step: one fused q/k/v GEMM -> ops.rotary_norm_store (norm, rotary,
cache write, all fp32 inside) -> ops.paged_attention over the block tables
of the batch (prompt portions and decode rows alike; every score map is a
"head" of the kernel) -> ops.diff_combine where there are two maps -> output
GEMM. This step's rows are read back from the pool like older positions.
"""
from __future__ import annotations

import math

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import PagedMixerSpec


class PagedRotaryAttention(nn.Module):
    def __init__(self, width: int, m: PagedMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "paged rotary attention is not sharded for tensor "
                "parallelism yet")
        if m.maps not in (1, 2):
            raise ValueError("one or two score maps per head")
        self.m, self.eps, self.comm = m, eps, comm
        self.nq = m.heads * m.maps * m.qk_dim
        self.nk = m.kv_heads * m.maps * m.qk_dim
        self.nv = 0 if m.tied_values else m.kv_heads * m.v_dim
        self.vw = m.v_width
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        n = self.nq + self.nk + self.nv
        self.qkv_w = mk(n, width)
        self.qkv_b = mk(n) if m.bias else None
        self.o_w = mk(width, m.heads * self.vw)
        f32 = torch.float32
        self.q_norm = mk(self.nq, dt=f32) if m.qk_norm_full else None
        self.k_norm = mk(self.nk, dt=f32) if m.qk_norm_full else None
        self.sinks = mk(m.heads, dt=f32) if m.sink else None
        # rows: lq1, lk1, lq2, lk2
        self.lam_vecs = mk(4, m.qk_dim, dt=f32) if m.maps == 2 else None
        self.register_buffer(
            "inv_freq", torch.tensor(m.rot.inv_freq(), dtype=torch.float64)
            .to(f32), persistent=False)
        self.register_buffer("lam", torch.zeros(1, dtype=f32),
                             persistent=False)

    def post_load(self) -> None:
        """Constants derived from loaded weights."""
        if self.lam_vecs is not None:
            v = self.lam_vecs.float()
            lam = (math.exp(float((v[0] * v[1]).sum()))
                   - math.exp(float((v[2] * v[3]).sum())) + self.m.diff)
            self.lam.fill_(lam)

    def forward(self, h, meta, k_cache, v_cache):
        m = self.m
        T = h.shape[0]
        rg = meta.ragged
        qkv = F.linear(h, self.qkv_w, self.qkv_b)
        q = torch.empty(T, self.nq, dtype=h.dtype, device=h.device)
        ops.rotary_norm_store(q, qkv, self.nq, self.nk, self.q_norm,
                              self.k_norm, self.inv_freq, rg.pos32, m.qk_dim,
                              k_cache, v_cache, meta.slot_mapping, self.eps,
                              m.tied_values,
                              page_groups=rg.page_groups(k_cache.shape[2])
                              if h.is_cuda and k_cache.shape[2] == 16
                              else None)
        A = m.heads * m.maps
        # two maps meet again in fp32 (their difference cancels digits)
        a = torch.empty(T, A, self.vw, device=h.device,
                        dtype=torch.float32 if m.maps == 2 else h.dtype)
        ops.paged_attention(
            a, q.view(T, A, m.qk_dim), k_cache, v_cache, rg.block_tables,
            rg.row_seq, rg.pos32, m.scale, maps=m.maps, window=m.window,
            keep_first=m.keep_first, sinks=self.sinks,
            tiles=rg.attn_tiles(m.heads, m.kv_heads, m.maps) if h.is_cuda
            else None, max_ctx=rg.max_ctx)
        if m.maps == 2:
            o = torch.empty(T, m.heads * self.vw, dtype=h.dtype,
                            device=h.device)
            ops.diff_combine(o, a.view(T, m.heads, 2, self.vw), self.lam,
                             m.diff, self.eps)
        else:
            o = a.view(T, A * self.vw)
        out = F.linear(o, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out
