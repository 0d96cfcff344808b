"""HIP kernels of the paged rotary attention family against their plain
PyTorch fp32 references (gpustack_amd/ops/torch_ref.py), on sizes that are
not multiples of a wave, a tile or a page, with windows, kept first keys,
sinks, two score maps and grouped heads, in prompts, decode rows and mixed
batches, on both the fp32 vector-ALU path and the MFMA path."""
import pytest
import torch

from gpustack_amd import ops
from gpustack_amd.ops import torch_ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(*shape, dtype=torch.float32, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * std).to(dtype).to(DEV)


@pytest.mark.parametrize("a_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [24, 30, 192, 1300, 1301, 5000, 9001])
def test_sandwich_add_norm(a_dtype, h_dtype, W):
    T = 19
    x = _rand(T, W)
    a = _rand(T, W, dtype=a_dtype, std=3.0, seed=2)
    pw, nw, ex = _rand(W, seed=3), _rand(W, seed=4), _rand(T, W, seed=5)
    for use_a, use_ex, use_next in [(1, 0, 1), (1, 1, 1), (0, 0, 1), (1, 1, 0),
                                    (0, 1, 1)]:
        xx, rx = x.clone(), x.clone()
        h = torch.zeros(T, W, dtype=h_dtype, device=DEV)
        rh = torch.zeros_like(h)
        args = (a if use_a else None, pw if use_a else None, 0.37, 1e-5,
                ex if use_ex else None, nw if use_next else None,
                None if not use_next else h)
        ops.sandwich_add_norm(xx, *args)
        rargs = args[:-1] + (None if not use_next else rh,)
        torch_ref.sandwich_add_norm(rx, *rargs)
        torch.testing.assert_close(xx, rx, rtol=1e-5, atol=1e-5)
        tol = 0.05 if h_dtype == torch.bfloat16 else 1e-4
        assert (h.float() - rh.float()).abs().max() <= tol


def test_embed_rows_and_act_and_mul():
    for dt in (torch.bfloat16, torch.float32):
        emb = _rand(50, 72, dtype=dt)
        tok = torch.randint(0, 50, (33,), device=DEV)
        x = torch.empty(33, 72, device=DEV)
        ops.embed_rows_f32(x, tok, emb)
        assert torch.equal(x, emb[tok].float())
        for F in (56, 52):          # 16-byte path and the scalar one
            gu = _rand(21, 2 * F, dtype=dt, std=2.0)
            for mode in ("gelu_tanh", "silu", "relu2", "gelu"):
                out = torch.empty(21, F, dtype=dt, device=DEV)
                ref = torch.empty_like(out)
                ops.act_and_mul(out, gu, mode)
                torch_ref.act_and_mul(ref, gu, mode)
                tol = 0.06 if dt == torch.bfloat16 else 1e-4
                assert (out.float() - ref.float()).abs().max() <= tol


def test_diff_combine():
    a = _rand(13, 5, 2, 40, std=2.0)
    lam = torch.tensor([0.83], device=DEV)
    for dt in (torch.bfloat16, torch.float32):
        out = torch.empty(13, 200, dtype=dt, device=DEV)
        ref = torch.empty_like(out)
        ops.diff_combine(out, a, lam, 0.3, 1e-5)
        torch_ref.diff_combine(ref, a, lam, 0.3, 1e-5)
        tol = 0.02 if dt == torch.bfloat16 else 1e-5
        assert (out.float() - ref.float()).abs().max() <= tol


def _pools(nb, G, KW, VW, dt):
    return (torch.zeros(nb, G, 16, KW, dtype=dt, device=DEV),
            torch.zeros(nb, G, VW, 16, dtype=dt, device=DEV))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("cfg", [
    # heads, kv, maps, D, VW, rot dims, full norm, tied
    (4, 2, 2, 24, 40, 8, False, False),
    (6, 3, 1, 20, 20, 20, True, True),
    (2, 2, 1, 64, 32, 0, False, False),
    # every width a multiple of 8: the 16-byte path for bf16
    (8, 2, 1, 64, 64, 32, True, True),
    (4, 2, 2, 32, 64, 12, False, False),
])
def test_rotary_norm_store(dt, cfg):
    H, G, maps, D, VW, rot, norm, tied = cfg
    T, nb = 37, 9
    nq, nk = H * maps * D, G * maps * D
    nv = 0 if tied else G * VW
    if tied:
        VW = maps * D
    qkv = _rand(T, nq + nk + nv, dtype=dt, std=1.5)
    qw = _rand(nq, seed=1) if norm else None
    kw = _rand(nk, seed=2) if norm else None
    inv = torch.tensor([10000.0 ** (-2 * i / max(rot, 1)) for i in range(rot // 2)],
                       dtype=torch.float32, device=DEV)
    pos = torch.randint(0, 3000, (T,), dtype=torch.int32, device=DEV)
    slots = torch.randperm(nb * 16, device=DEV)[:T].long()
    slots[5] = -1
    kc, vc = _pools(nb, G, maps * D, VW, dt)
    rkc, rvc = kc.clone(), vc.clone()
    q = torch.empty(T, nq, dtype=dt, device=DEV)
    rq = torch.empty_like(q)
    ops.rotary_norm_store(q, qkv, nq, nk, qw, kw, inv, pos, D, kc, vc, slots,
                          1e-5, tied)
    torch_ref.rotary_norm_store(rq, qkv, nq, nk, qw, kw, inv, pos, D, rkc, rvc,
                                slots, 1e-5, tied)
    # angles reach thousands of radians: fp32 sin/cos of the same fp32
    # angle, so only the last bits differ
    tol = 0.05 if dt == torch.bfloat16 else 2e-4
    assert (q.float() - rq.float()).abs().max() <= tol
    assert (kc.float() - rkc.float()).abs().max() <= tol
    assert torch.equal(vc, rvc)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tied", [False, True])
def test_value_rows_stored_page_by_page(dt, tied):
    """Prompt portions that start and end inside pages: whole pages leave
    in one piece, the ragged ends and single rows one store at a time."""
    H, G, D = 4, 2, 32
    VW = D if tied else 72
    seqs = [(0, 40), (5, 1), (30, 51), (16, 16), (47, 2)]
    nb = sum((h + n + 15) // 16 for h, n in seqs) + 1
    perm = torch.randperm(nb).tolist()
    starts, hists, news, slots, pos = [], [], [], [], []
    for h, n in seqs:
        blocks = [perm.pop() for _ in range((h + n + 15) // 16)]
        starts.append(len(pos)); hists.append(h); news.append(n)
        pos += list(range(h, h + n))
        slots += [blocks[p // 16] * 16 + p % 16 for p in range(h, h + n)]
    T = len(pos)
    nq, nk = H * D, G * D
    qkv = _rand(T, nq + nk + (0 if tied else G * VW), dtype=dt, std=1.5)
    inv = torch.tensor([100.0 ** (-i / 8) for i in range(8)], device=DEV)
    pos = torch.tensor(pos, dtype=torch.int32, device=DEV)
    slots = torch.tensor(slots, device=DEV)
    kc, vc = _pools(nb, G, D, VW, dt)
    vc.fill_(7.0)
    rkc, rvc = kc.clone(), vc.clone()
    q, rq = (torch.empty(T, nq, dtype=dt, device=DEV) for _ in range(2))
    groups = ops.build_page_groups(starts, hists, news, 16, DEV)
    assert int(groups[:, 1].sum()) == T and int(groups[:, 1].max()) == 16
    ops.rotary_norm_store(q, qkv, nq, nk, None, None, inv, pos, D, kc, vc, slots,
                          1e-5, tied, page_groups=groups)
    torch_ref.rotary_norm_store(rq, qkv, nq, nk, None, None, inv, pos, D, rkc,
                                rvc, slots, 1e-5, tied)
    assert torch.equal(vc, rvc)
    assert (kc.float() - rkc.float()).abs().max() <= 0.05


def _attn_case(dt, H, G, maps, D, VW, window, keep, sink, seqs, exact,
               seed=0):
    """seqs: list of (cached tokens, new rows). Fills the pools for every
    position, then runs the new rows of all sequences as one batch."""
    torch.manual_seed(seed)
    A = H * maps
    nb = sum((h + n + 15) // 16 for h, n in seqs) + 2
    kc, vc = _pools(nb, G, maps * D, VW, dt)
    kc.copy_(torch.randn(kc.shape, device=DEV).to(dt))
    vc.copy_(torch.randn(vc.shape, device=DEV).to(dt))
    perm = torch.randperm(nb - 1).tolist()
    maxb = max((h + n + 15) // 16 for h, n in seqs)
    bt = torch.zeros(len(seqs), maxb, dtype=torch.int32)
    starts, hists, news, row_seq, pos = [], [], [], [], []
    for i, (h, n) in enumerate(seqs):
        k = (h + n + 15) // 16
        bt[i, :k] = torch.tensor([perm.pop() for _ in range(k)])
        starts.append(len(pos)); hists.append(h); news.append(n)
        row_seq += [i] * n
        pos += list(range(h, h + n))
    T = len(pos)
    q = (torch.randn(T, A, D, device=DEV) * 1.5).to(dt)
    sinks = torch.randn(H, device=DEV) if sink else None
    bt = bt.to(DEV)
    row_seq = torch.tensor(row_seq, dtype=torch.int32, device=DEV)
    pos = torch.tensor(pos, dtype=torch.int32, device=DEV)
    tiles = ops.build_attn_tiles(starts, hists, news, H, G, maps, DEV)
    odt = torch.float32 if (maps == 2 or dt == torch.float32) else dt
    out = torch.zeros(T, A, VW, dtype=odt, device=DEV)
    ops.paged_attention(out, q, kc, vc, bt, row_seq, pos, 0.21, maps=maps,
                        window=window, keep_first=keep, sinks=sinks,
                        tiles=tiles, exact=exact,
                        max_ctx=max(h + n for h, n in seqs))
    ref = torch.zeros(T, A, VW)
    torch_ref.paged_attention(ref, q.cpu(), kc.cpu(), vc.cpu(), bt.cpu(),
                              row_seq.cpu(), pos.cpu(), 0.21, maps, window,
                              keep, sinks.cpu() if sink else None)
    return out.float().cpu(), ref


MIXED = [(0, 37), (130, 1), (45, 19), (700, 1), (16, 16), (31, 2)]


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", [
    # H, G, maps, D, VW, window, keep_first, sink
    (4, 2, 2, 24, 40, 50, 3, False),
    (3, 3, 1, 20, 20, 0, 0, True),
    (8, 2, 1, 64, 96, 33, 0, True),
    (2, 1, 2, 32, 16, 0, 0, False),
])
def test_paged_attention_exact(dt, shape):
    out, ref = _attn_case(dt, *shape, seqs=MIXED, exact=True)
    assert (out - ref).abs().max() <= (2e-2 if dt == torch.bfloat16 else 2e-4)


@pytest.mark.parametrize("shape", [
    (6, 3, 2, 32, 48, 100, 5, False),
    (4, 4, 1, 128, 128, 0, 0, True),
    (8, 2, 1, 64, 96, 70, 20, True),
    (6, 2, 2, 96, 48, 0, 0, False),
])
@pytest.mark.parametrize("seqs", [MIXED, [(0, 300)], [(1500, 1), (2100, 1)],
                                  [(600, 3)]])
def test_paged_attention_mfma(shape, seqs):
    """bf16 q and pools of fitting sizes take the MFMA kernel (key split +
    merge for the long decode rows); weights are rounded to bf16 for the
    second product, so the tolerance is bf16-sized."""
    out, ref = _attn_case(torch.bfloat16, *shape, seqs=seqs, exact=False)
    assert (out - ref).abs().max() <= 3e-2
