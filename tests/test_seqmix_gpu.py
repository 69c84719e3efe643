"""HIP sequence-mixer kernels against the PyTorch fp32 implementations of
the same ops (ops/seqmix_reference.py), in fp32 and bf16, on shapes that
are not multiples of the tile sizes."""

import math

import pytest
import torch

from fusioninfer_amd.ops import seqmix
from fusioninfer_amd.ops import seqmix_reference as ref

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]


def tol(dtype):
    return dict(atol=2e-5, rtol=2e-5) if dtype == torch.float32 else \
        dict(atol=3e-2, rtol=3e-2)


def groups(lens, pos0, slots, dev):
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    row_seq = [s for s, n in enumerate(lens) for _ in range(n)]
    positions = [pos0[s] + i for s, n in enumerate(lens) for i in range(n)]
    mk = lambda x: torch.tensor(x, dtype=torch.int32, device=dev)
    return mk(cu), mk(row_seq), mk(positions), mk(slots)


@pytest.fixture(autouse=True)
def _native():
    assert seqmix.has_native(), "sequence-mixer extension not built"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("W", [96, 256, 1000, 37, 2050])
def test_row_norms(dtype, W):
    torch.manual_seed(0)
    dev = "cuda"
    T = 37
    x = torch.randn(T, W, device=dev) * 3
    g = torch.tensor([1.3], device=dev)
    g2 = torch.tensor([0.7], device=dev)
    out = seqmix.scalar_rms_norm(x, g, 1e-5, dtype)
    exp = ref.scalar_rms_norm(x.cpu(), g.cpu(), 1e-5, dtype)
    torch.testing.assert_close(out.cpu().float(), exp.float(), **tol(dtype))

    y = (torch.randn(T, W, device=dev) * 2).to(dtype)
    for gn in (None, g2):
        r1, r2 = x.clone(), x.cpu().clone()
        h1 = seqmix.residual_add_scalar_norm_(r1, y, g, 1e-5, gn, dtype)
        h2 = ref.residual_add_scalar_norm_(r2, y.cpu(), g.cpu(), 1e-5,
                                           None if gn is None else gn.cpu(),
                                           dtype)
        torch.testing.assert_close(r1.cpu(), r2, atol=2e-5, rtol=2e-5)
        if gn is not None:
            torch.testing.assert_close(h1.cpu().float(), h2.float(),
                                       **tol(dtype))

    yl = (torch.randn(T, W, device=dev)).to(dtype)
    yr = (torch.randn(T, W, device=dev) * 5).to(dtype)
    wl, wr = torch.rand(W, device=dev) + 0.5, torch.rand(W, device=dev) + 0.5
    for gn in (None, g2):
        r1, r2 = x.clone(), x.cpu().clone()
        h1 = seqmix.dual_norm_combine_residual_(r1, yl, yr, wl, wr, g, 1e-5,
                                                gn, dtype)
        h2 = ref.dual_norm_combine_residual_(
            r2, yl.cpu(), yr.cpu(), wl.cpu(), wr.cpu(), g.cpu(), 1e-5,
            None if gn is None else gn.cpu(), dtype)
        torch.testing.assert_close(r1.cpu(), r2, atol=2e-5, rtol=2e-5)
        if gn is not None:
            torch.testing.assert_close(h1.cpu().float(), h2.float(),
                                       **tol(dtype))

    gu = torch.randn(T, 2 * W, device=dev).to(dtype) * 2
    torch.testing.assert_close(
        seqmix.gelu_tanh_and_mul(gu).cpu().float(),
        ref.gelu_tanh_and_mul(gu.cpu()).float(), **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
def test_norm_token_shift_groups_and_slots(dtype):
    torch.manual_seed(1)
    dev = "cuda"
    W = 200
    lens, pos0, slots = [5, 1, 1, 7, 2], [0, 9, 0, 3, 0], [2, 0, -1, 3, 1]
    cu, row_seq, positions, sl = groups(lens, pos0, slots, dev)
    T = sum(lens)
    x = torch.randn(T, W, device=dev)
    g = torch.tensor([0.9], device=dev)
    shift = torch.rand(W, device=dev)
    state = torch.randn(5, W, device=dev)
    s1, s2 = state.clone(), state.cpu().clone()
    o1 = seqmix.norm_token_shift(x, g, shift, s1, cu, row_seq, positions, sl,
                                 1e-5, dtype)
    o2 = ref.norm_token_shift(x.cpu(), g.cpu(), shift.cpu(), s2, cu.cpu(),
                              row_seq.cpu(), positions.cpu(), sl.cpu(), 1e-5,
                              dtype)
    torch.testing.assert_close(o1.cpu().float(), o2.float(), **tol(dtype))
    torch.testing.assert_close(s1.cpu(), s2, atol=2e-5, rtol=2e-5)
    # the untouched slot keeps its content
    assert torch.equal(s1[4], state[4])


def _fill_cache(dtype, lens_total, G, D, bs, dev, seed):
    """Random block tables (shuffled physical blocks) for sequences."""
    g = torch.Generator().manual_seed(seed)
    nb = sum((n + bs - 1) // bs for n in lens_total) + 3
    perm = torch.randperm(nb, generator=g).tolist()
    bts, width = [], max((n + bs - 1) // bs for n in lens_total)
    for n in lens_total:
        k = (n + bs - 1) // bs
        bts.append([perm.pop() for _ in range(k)] + [0] * (width - k))
    kc = torch.zeros(nb, G, bs, D, dtype=dtype, device=dev)
    vc = torch.zeros(nb, G, bs, D, dtype=dtype, device=dev)
    return kc, vc, torch.tensor(bts, dtype=torch.int32, device=dev)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,D,rot", [(4, 2, 64, 64), (3, 3, 80, 32),
                                       (8, 1, 128, 0), (2, 2, 30, 30),
                                       (2, 1, 96, 40), (2, 2, 32, 32),
                                       (1, 1, 256, 64)])
def test_rope_unitnorm_cache_and_attention(dtype, H, G, D, rot):
    torch.manual_seed(2)
    dev = "cuda"
    bs = 16
    lens, pos0 = [140, 1, 9, 1], [0, 130, 57, 0]
    total = [p + n for p, n in zip(pos0, lens)]
    kc, vc, bt = _fill_cache(dtype, total, G, D, bs, dev, 3)
    # earlier context of every sequence: random processed/raw keys
    kc.copy_(torch.randn(kc.shape, device=dev).to(dtype))
    vc.copy_(torch.randn(vc.shape, device=dev).to(dtype))
    cu, row_seq, positions, _ = groups(lens, pos0, [0] * 4, dev)
    T = sum(lens)
    slot_map = []
    for s, n in enumerate(lens):
        for i in range(n):
            p = pos0[s] + i
            slot_map.append(int(bt[s, p // bs]) * bs + p % bs)
    slot_map = torch.tensor(slot_map, dtype=torch.int32, device=dev)
    proj = torch.randn(T, (H + G) * D + 5, device=dev).to(dtype)
    q, k = proj[:, : H * D], proj[:, H * D: (H + G) * D]
    from fusioninfer_amd.models.mixers import rotary_inv_freq

    inv = rotary_inv_freq(rot, 10000.0).to(dev)
    kc2, vc2 = kc.cpu().clone(), vc.cpu().clone()
    qn = seqmix.rope_unitnorm_cache_(q, k, positions, inv, 1e-5, kc, vc,
                                     slot_map, H, G, D)
    qn2 = ref.rope_unitnorm_cache_(q.cpu(), k.cpu(), positions.cpu(),
                                   inv.cpu(), 1e-5, kc2, vc2, slot_map.cpu(),
                                   H, G, D)
    torch.testing.assert_close(qn.cpu().float().view(T, H, D), qn2.float().view(T, H, D),
                               **tol(dtype))
    torch.testing.assert_close(kc.cpu().float(), kc2.float(), **tol(dtype))
    assert torch.equal(vc.cpu(), vc2)
    all_tiles = seqmix.build_attention_tiles(lens, device=dev)
    lead_tiles = seqmix.build_attention_tiles(lens[:1], device=dev)
    for chunk, window in [(0, 0), (50, 0), (0, 33), (64, 20)]:
        o2 = ref.ranged_paged_attention(
            qn.cpu().view(T, H, D), kc.cpu(), vc.cpu(), bt.cpu(),
            row_seq.cpu(), positions.cpu(), 0.2, chunk, window)
        # row-per-wave kernel; tiled kernel on every group; tiled kernel
        # on the leading group and rows for the rest
        for tiles in (None, all_tiles, lead_tiles):
            o1 = seqmix.ranged_paged_attention(
                qn.view(T, H, D), kc, vc, bt, row_seq, positions, 0.2, chunk,
                window, seq_cu=cu, tiles=tiles)
            torch.testing.assert_close(o1.cpu().float(), o2.float(),
                                       **tol(dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim", [(2, 64), (3, 48), (1, 128), (2, 16)])
def test_delta_rule(dtype, heads, dim):
    torch.manual_seed(4)
    dev = "cuda"
    n = heads * dim
    lens, pos0, slots = [33, 1, 1, 6], [0, 12, 0, 5], [1, 3, -1, 0]
    cu, row_seq, positions, sl = groups(lens, pos0, slots, dev)
    T = sum(lens)
    proj = torch.randn(T, 6 * n + 3, device=dev).to(dtype)
    r, k, v, wl, al, gl = [proj[:, i * n: (i + 1) * n] for i in range(6)]
    w0 = torch.randn(n, device=dev)
    ab = torch.randn(n, device=dev)
    nw = torch.rand(n, device=dev) + 0.5
    state = torch.randn(4, heads, dim, dim, device=dev) * 0.3
    s1, s2 = state.clone(), state.cpu().clone()
    o1 = seqmix.delta_rule(r, k, v, wl, al, gl, w0, ab, nw, s1, cu, sl,
                           positions, heads, dim, 1e-5, math.exp(-0.5))
    o2 = ref.delta_rule(r.cpu(), k.cpu(), v.cpu(), wl.cpu(), al.cpu(),
                        gl.cpu(), w0.cpu(), ab.cpu(), nw.cpu(), s2, cu.cpu(),
                        sl.cpu(), positions.cpu(), heads, dim, 1e-5,
                        math.exp(-0.5))
    torch.testing.assert_close(o1.cpu().float(), o2.float(), **tol(dtype))
    torch.testing.assert_close(s1.cpu(), s2, atol=1e-4, rtol=1e-4)
    assert torch.equal(s1[2], state[2])
