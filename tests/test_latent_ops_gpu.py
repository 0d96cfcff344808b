"""HIP kernels of the fp32-residual op family against their plain PyTorch
fp32 references (gpustack_amd/ops/torch_ref.py), on sizes that are not
multiples of a wave, a tile or a page."""
import pytest
import torch

from gpustack_amd import ops
from gpustack_amd.ops import torch_ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(*shape, dtype=torch.float32, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * std).to(dtype).to(DEV)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [40, 192, 1000])
def test_embed_pair_hash(dtype, W):
    V, B, T = 77, 13, 29
    emb, pair = _rand(V, W, dtype=dtype), _rand(B + 1, W, dtype=dtype, seed=1)
    tok = torch.randint(0, V, (T,), device=DEV)
    prev = torch.randint(0, V, (T,), device=DEV)
    prev[[0, 7]] = -1
    x = torch.empty(T, W, device=DEV)
    h = torch.empty(T, W, dtype=dtype, device=DEV) if dtype == torch.bfloat16 else None
    ops.embed_pair_hash(x, h, tok, prev, emb, pair, B, 19, 3)
    rx = torch.empty_like(x)
    rh = torch.empty_like(h) if h is not None else None
    torch_ref.embed_pair_hash(rx, rh, tok, prev, emb, pair, B, 19, 3)
    assert torch.equal(x, rx)
    if h is not None:
        assert torch.equal(h, rh)
    # no pair table at all
    ops.embed_pair_hash(x, h, tok, prev, emb, None, 0, 0, 0)
    assert torch.equal(x, emb[tok].float())


@pytest.mark.parametrize("a_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [24, 192, 777])
def test_rms_scale_add_and_norm(a_dtype, W):
    T = 19
    x = _rand(T, W)
    a = _rand(T, W, dtype=a_dtype, std=3.0, seed=2)
    w, s = _rand(W, seed=3), _rand(W, seed=4)
    for scale in (s, None):
        xx, rx = x.clone(), x.clone()
        h = torch.empty(T, W, dtype=torch.bfloat16, device=DEV)
        rh = torch.empty_like(h)
        ops.rms_scale_add(xx, a, w, scale, 1e-5, h)
        torch_ref.rms_scale_add(rx, a, w, scale, 1e-5, rh)
        torch.testing.assert_close(xx, rx, rtol=1e-5, atol=1e-5)
        assert (h.float() - rh.float()).abs().max() <= 0.05
    for od in (torch.bfloat16, torch.float32):
        out = torch.empty(T, W, dtype=od, device=DEV)
        ref = torch.empty_like(out)
        ops.rms_norm_f32(out, x, w, 1e-6)
        torch_ref.rms_norm_f32(ref, x, w, 1e-6)
        torch.testing.assert_close(out.float(), ref.float(), rtol=1e-2 if od == torch.bfloat16 else 1e-5, atol=1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("T,NB", [(21, 5), (300, 20)])   # row / 16-row kernels
@pytest.mark.parametrize("R,col0,pad", [(72, 50, 6), (72, 48, 8), (512, 64, 0)])
def test_latent_norm_store(dtype, T, NB, R, col0, pad):
    BS = 16    # (72, 48, 8) and (512, 64, 0): 16-byte aligned bf16 rows
    src = _rand(T, col0 + R + pad, dtype=dtype, std=2.0)
    w = _rand(R, seed=5)
    slots = torch.randperm(NB * BS)[:T].to(DEV)
    slots[3] = -1
    if T >= 64:
        # rows 16..47 fill two whole pages in order (vector store path),
        # rows 0..15 fill a page backwards, the rest is scattered
        n = NB * BS
        keep = torch.ones(n, dtype=torch.bool)
        keep[32:64] = False
        keep[n - 16:] = False
        free = torch.nonzero(keep).flatten()
        slots = torch.cat([torch.arange(n - 1, n - 17, -1),
                           torch.arange(32, 64),
                           free[torch.randperm(len(free))[:T - 48]]]).to(DEV)
        slots[50] = -1
    for planes in (1, 2):
        cache = torch.zeros(NB, planes, BS, R, dtype=dtype, device=DEV)
        ref = torch.zeros_like(cache)
        ops.latent_norm_store(cache, src, col0, w, slots, 1e-6)
        torch_ref.latent_norm_store(ref, src, col0, w, slots, 1e-6)
        torch.testing.assert_close(
            cache.float(), ref.float(),
            rtol=1e-2 if dtype == torch.bfloat16 else 1e-5, atol=1e-5)
        if planes == 2:   # plane 1 is plane 0 transposed, page by page
            assert torch.equal(cache[:, 1].reshape(NB, R, BS).transpose(1, 2),
                               cache[:, 0])


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mode", ["relu2", "gelu", "gelu_tanh", "silu"])
def test_act_inplace(dtype, mode):
    x = _rand(37, 51, dtype=dtype, std=2.0)
    ref = x.clone()
    ops.act_inplace(x, mode)
    torch_ref.act_inplace(ref, mode)
    torch.testing.assert_close(x.float(), ref.float(),
                               rtol=1e-2 if dtype == torch.bfloat16 else 1e-5,
                               atol=1e-5)


@pytest.mark.parametrize("E,G,keep,top", [(10, 5, 3, 4), (12, 1, 1, 3),
                                          (96, 8, 2, 6), (130, 5, 5, 7)])
def test_route_grouped_topk(E, G, keep, top):
    T = 41
    logits = _rand(T, E + 1, std=2.0)
    ex = torch.empty(T, top, dtype=torch.int32, device=DEV)
    wt = torch.empty(T, top, device=DEV)
    rex, rwt = torch.empty_like(ex), torch.empty_like(wt)
    ops.route_grouped_topk(ex, wt, logits, E, G, keep, 1.75)
    torch_ref.route_grouped_topk(rex, rwt, logits, E, G, keep, 1.75)
    assert torch.equal(ex.sort(1)[0], rex.sort(1)[0])
    torch.testing.assert_close(wt.sort(1)[0], rwt.sort(1)[0], rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_moe_combine_softcap_argmax(dtype):
    T, W, top = 23, 100, 3
    y = _rand(T * top, W, dtype=dtype)
    inv = torch.randperm(T * top).to(torch.int32).view(T, top).to(DEV)
    wt = _rand(T, top, seed=6).abs()
    sh = _rand(T, W, dtype=dtype, seed=7)
    gate = _rand(T, 5, seed=8)
    for shared, g in ((sh, gate), (sh, None), (None, None)):
        out = torch.empty(T, W, device=DEV)
        ref = torch.empty_like(out)
        ops.moe_combine(out, y, inv, wt, shared, g, 4)
        torch_ref.moe_combine(ref, y, inv, wt, shared, g, 4)
        torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
    lg = _rand(9, 333, std=20.0)
    ref = 11.0 * torch.tanh(lg / 11.0)
    ops.softcap_(lg, 11.0)
    torch.testing.assert_close(lg, ref, rtol=1e-5, atol=1e-5)
    assert torch.equal(ops.greedy_sample(lg), lg.argmax(-1))


def _attention_case(dtype, H, R, BS, seqs, seed=0, planes=1, qstd=0.3):
    """seqs: list of (hist, new). Builds a shuffled paged pool."""
    g = torch.Generator().manual_seed(seed)
    nblk = sum((h + n + BS - 1) // BS for h, n in seqs) + 2
    perm = torch.randperm(nblk - 1, generator=g).tolist()
    rows = torch.randn(nblk, BS, R, generator=g).to(dtype)
    cache = torch.stack([rows] + [rows.transpose(1, 2).reshape(nblk, BS, R)]
                        * (planes - 1), dim=1).contiguous().to(DEV)
    maxb = max((h + n + BS - 1) // BS for h, n in seqs)
    bt = torch.zeros(len(seqs), maxb, dtype=torch.int32)
    starts, hists, news, row_seq, pos = [], [], [], [], []
    off = 0
    for i, (h, n) in enumerate(seqs):
        nb = (h + n + BS - 1) // BS
        bt[i, :nb] = torch.tensor([perm.pop() for _ in range(nb)])
        starts.append(off); hists.append(h); news.append(n)
        row_seq += [i] * n
        pos += list(range(h, h + n))
        off += n
    T = off
    q = (torch.randn(T, H, R, generator=g) * qstd).to(DEV)
    return (cache, bt.to(DEV), torch.tensor(row_seq, dtype=torch.int32, device=DEV),
            torch.tensor(pos, dtype=torch.int32, device=DEV), q,
            ops.build_latent_tiles(starts, hists, news, H, DEV))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,R", [(7, 88), (3, 40), (20, 200), (2, 520)])
def test_latent_attention(dtype, H, R):
    seqs = [(0, 37), (45, 1), (16, 16), (31, 2), (0, 1), (63, 70)]
    cache, bt, row_seq, pos, q, tiles = _attention_case(dtype, H, R, 16, seqs)
    ctx = torch.empty_like(q)
    ops.latent_attention(ctx, q, cache, bt, row_seq, pos, 0.2, tiles=tiles,
                         exact=True)
    ref_c = torch.empty_like(q.cpu())
    torch_ref.latent_attention(ref_c, q.cpu(), cache.cpu(), bt.cpu(),
                               row_seq.cpu(), pos.cpu(), 0.2)
    torch.testing.assert_close(ctx.cpu(), ref_c, rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("H,R", [(3, 96), (1, 32), (16, 128), (5, 512),
                                 (3, 1024), (20, 64)])
def test_latent_attention_mfma(H, R):
    """bf16 two-plane pool: the MFMA kernel against the fp32 reference (it
    rounds the scaled query and the softmax weights to bf16) and against
    the exact kernel on the same pool."""
    seqs = [(0, 37), (45, 1), (16, 16), (31, 2), (0, 1), (63, 70), (200, 3),
            (0, 130)]
    cache, bt, row_seq, pos, q, tiles = _attention_case(
        torch.bfloat16, H, R, 16, seqs, planes=2, qstd=1.0 / R ** 0.5)
    assert ops._load_latent().latent_attention_uses_mfma(cache)
    ctx, ex = torch.empty_like(q), torch.empty_like(q)
    ops.latent_attention(ctx, q, cache, bt, row_seq, pos, 1.0, tiles=tiles)
    ops.latent_attention(ex, q, cache, bt, row_seq, pos, 1.0, tiles=tiles,
                         exact=True)
    ref = torch.empty_like(q.cpu())
    torch_ref.latent_attention(ref, q.cpu(), cache.cpu(), bt.cpu(),
                               row_seq.cpu(), pos.cpu(), 1.0)
    torch.testing.assert_close(ex.cpu(), ref, rtol=2e-4, atol=2e-5)
    err = (ctx.cpu() - ref).abs().max().item()
    assert err < 0.03, err
    assert ops.latent_attention_mfma_ok(cache)
    # keys split over several workgroups and merged
    sp = torch.empty_like(q)
    ops._load_latent().latent_attention(sp, q, cache, bt, tiles, pos, 1.0,
                                        False, 5)
    assert (sp.cpu() - ref).abs().max().item() < 0.03
    # bf16 operands in head-major buffers, passed as strided [T, H, R] views
    T = q.shape[0]
    qb = q.to(torch.bfloat16).transpose(0, 1).contiguous()
    for nsplit in (1, 3):
        ob = torch.full((H, T, R), float("nan"), dtype=torch.bfloat16, device=DEV)
        ops._load_latent().latent_attention(ob.transpose(0, 1), qb.transpose(0, 1),
                                            cache, bt, tiles, pos, 1.0, False,
                                            nsplit)
        got = ob.transpose(0, 1).float().cpu()
        assert (got - ref).abs().max().item() < 0.05


def test_latent_attention_mfma_one_far_key_decides():
    """Scale each query so that ONE key far back (the first positions, both
    sides of page borders, the row's own position) takes the whole softmax:
    the output must be that key's latent."""
    H, R, BS = 4, 64, 16
    hist = 300
    targets = [0, 1, 15, 16, 17, 31, 32, 63, 64, 255, 256, 287, 288, 299, 300]
    seqs = [(hist, 1)] * len(targets) + [(0, 301)]
    cache, bt, row_seq, pos, q, tiles = _attention_case(
        torch.bfloat16, H, R, BS, seqs, planes=2)
    T = q.shape[0]
    want = torch.empty(T, H, R)
    rows = list(range(len(targets))) + [T - 1]
    tg = targets + [123]
    for row, j in zip(rows, tg):
        s = int(row_seq[row])
        c = cache[bt[s, j // BS].long(), 0, j % BS].float()
        q[row] = 40.0 * c / c.norm()
        want[row] = c.cpu()
    for exact in (False, True):
        ctx = torch.empty_like(q)
        ops.latent_attention(ctx, q, cache, bt, row_seq, pos, 1.0, tiles=tiles,
                             exact=exact)
        torch.testing.assert_close(ctx.cpu()[rows], want[rows],
                                   rtol=0.02, atol=0.02)
