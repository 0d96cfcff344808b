"""Position-free latent attention mixer.

Every token leaves ONE RMS-normalised latent c (width R) in the paged pool;
head a's keys and values are the linear images U_k[a] c and U_v[a] c. No
rotation or other positional signal enters the scores, so — unlike the
DeepSeek-style MLAAttention in models/llama.py — there is no rope slice in
the cache row and the absorbed form is exact for the whole score:

    q~[t,a] = U_k[a]^T q[t,a]                       (width R, fp32)
    ctx[t,a] = softmax_{j<=pos(t)}(scale * q~[t,a] . c_j) . C
    out[t]   = W_o concat_a(U_v[a] ctx[t,a])

Only c is ever read per cached token (R values instead of
heads * (Dq + Dv)), by all heads of a row at once: ops.latent_attention
streams a sequence's latents once per 16 (row, head) pairs. Scores, the
softmax and the latent norm are fp32 in every engine dtype; head sizes,
latent width and score scale are constructor parameters.
"""
from __future__ import annotations

import torch
import torch.nn.functional as F
from torch import nn

from .. import ops
from ..engine.config import LatentMixerSpec


class LatentAttention(nn.Module):
    def __init__(self, width: int, m: LatentMixerSpec, eps: float, dtype,
                 comm=None):
        super().__init__()
        if comm is not None and comm.tp_size > 1:
            raise NotImplementedError(
                "latent attention is not sharded for tensor parallelism yet")
        self.comm = comm
        self.h, self.dq, self.dv, self.r = m.heads, m.qk_dim, m.v_dim, m.kv_rank
        self.scale = float(m.scale)
        self.eps = eps
        mk = lambda *shape, dt=dtype: nn.Parameter(
            torch.empty(*shape, dtype=dt), requires_grad=False)
        # q and the latent down-projection fused: one GEMM per layer entry
        self.qd_w = mk(self.h * self.dq + self.r, width)
        self.lat_norm = mk(self.r, dt=torch.float32)
        # absorbed factors, head-major, in the GEMM dtype (fp32 engines keep
        # every product fp32; bf16 engines feed the MFMA kernel, which
        # rounds q~ to bf16 anyway)
        self.uk = mk(self.h, self.dq, self.r)
        self.uv_t = mk(self.h, self.r, self.dv)
        self.o_w = mk(width, self.h * self.dv)

    def forward(self, h, meta, cache):
        T = h.shape[0]
        rg = meta.ragged
        nq = self.h * self.dq
        qd = F.linear(h, self.qd_w)                        # [T, H*Dq + R]
        # norm + cache write first: this step's rows are read back from
        # the pool like every earlier position
        ops.latent_norm_store(cache, qd, nq, self.lat_norm,
                              meta.slot_mapping, self.eps)
        q = qd[:, :nq].unflatten(1, (self.h, self.dq))     # [T, H, Dq]
        q_hts = torch.bmm(q.transpose(0, 1), self.uk)      # [H, T, R]
        if ops.latent_attention_mfma_ok(cache):
            # bf16 in, bf16 out, head-major buffers handed to the kernel as
            # strided [T, H, R] views: no transposing or casting passes
            # between the two batched projections and the kernel
            q_lat = q_hts.transpose(0, 1)
            ctx_hts = torch.empty(self.h, T, self.r, dtype=h.dtype,
                                  device=h.device)
            ctx = ctx_hts.transpose(0, 1)
        else:
            q_lat = q_hts.transpose(0, 1).float().contiguous()
            ctx = torch.empty(T, self.h, self.r, dtype=torch.float32,
                              device=h.device)
            ctx_hts = None
        ops.latent_attention(ctx, q_lat, cache, rg.block_tables, rg.row_seq,
                             rg.pos32, self.scale,
                             tiles=rg.latent_tiles(self.h) if h.is_cuda
                             else None, max_ctx=rg.max_ctx)
        if ctx_hts is None:
            ctx_hts = ctx.transpose(0, 1).to(self.uv_t.dtype)
        o = torch.bmm(ctx_hts, self.uv_t)                  # [H, T, Dv]
        o = o.transpose(0, 1).reshape(T, self.h * self.dv)  # [T, H*Dv]
        out = F.linear(o, self.o_w)
        return self.comm.all_reduce(out) if self.comm is not None else out
