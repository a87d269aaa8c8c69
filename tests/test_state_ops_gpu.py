"""HIP kernels of the layer-norm stream, the head-norm cache write, scored
routing and the recurrent mixers against their plain PyTorch fp32 references
(gpustack_amd/ops/torch_ref.py): sizes that are not multiples of a wave or
a page, ragged batches (portions, single rows, sequences that start at
position 0 and ones that resume from a slot), state sizes on both sides of
every lane split, and the distance slopes of the paged attention kernels."""
import pytest
import torch

from gpustack_amd import ops
from gpustack_amd.ops import torch_ref

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _rand(*shape, dtype=torch.float32, std=1.0, seed=0):
    g = torch.Generator().manual_seed(seed + sum(shape))
    return (torch.randn(*shape, generator=g) * std).to(dtype).to(DEV)


def _i32(v):
    return torch.tensor(v, dtype=torch.int32, device=DEV)


def _ragged(news, hists, slots):
    """seq_first, seq_rows, state_slots, row_seq, pos32 of a ragged batch."""
    first, rs, pos = [], [], []
    r = 0
    for i, (n, h) in enumerate(zip(news, hists)):
        first.append(r)
        rs += [i] * n
        pos += list(range(h, h + n))
        r += n
    return _i32(first), _i32(news), _i32(slots), _i32(rs), _i32(pos)


@pytest.mark.parametrize("a_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("h_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("W", [24, 30, 192, 1300, 2049, 5000])
def test_add_layer_norm(a_dtype, h_dtype, W):
    T = 13
    x = _rand(T, W, std=4.0) + 1.5
    a = _rand(T, W, dtype=a_dtype, std=3.0, seed=2)
    w, b = _rand(W, seed=3), _rand(W, seed=4)
    for use_a, use_n in [(1, 1), (0, 1), (1, 0)]:
        xx, rx = x.clone(), x.clone()
        h = torch.zeros(T, W, dtype=h_dtype, device=DEV)
        rh = torch.zeros_like(h)
        ops.add_layer_norm(xx, a if use_a else None, w if use_n else None,
                           b if use_n else None, 1e-5, h if use_n else None)
        torch_ref.add_layer_norm(rx, a if use_a else None,
                                 w if use_n else None, b if use_n else None,
                                 1e-5, rh if use_n else None)
        torch.testing.assert_close(xx, rx, rtol=1e-6, atol=1e-6)
        tol = 0.05 if h_dtype == torch.bfloat16 else 2e-4
        assert (h.float() - rh.float()).abs().max() <= tol


def test_embed_rows_scaled():
    for dt in (torch.bfloat16, torch.float32):
        emb = _rand(50, 72, dtype=dt)
        tok = torch.randint(0, 50, (33,), device=DEV)
        x = torch.empty(33, 72, device=DEV)
        ops.embed_rows_scaled(x, tok, emb, 7.5)
        assert torch.equal(x, emb[tok].float() * 7.5)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("mix", [False, True])
@pytest.mark.parametrize("paged", [False, True])
def test_head_norm_store(dtype, mix, paged):
    HQ, G, D, VW, BS, nb = 6, 3, 40, 24, 16, 9
    T = 37
    nq, nk, nv = HQ * D, G * D, G * VW
    qkv = _rand(T, nq + nk + nv, dtype=dtype, std=2.0)
    vf_src = _rand(T, nq + nk + nv, dtype=dtype, seed=9)
    v_first = vf_src[:, nq + nk:] if mix else None
    lam = torch.tensor([0.3], device=DEV)
    qw, kw = _rand(D, seed=1) + 1, _rand(D, seed=2) + 1
    pos = _i32([(5 * t) % 130 for t in range(T)])
    perm = torch.randperm(nb * BS)[:T].to(DEV)
    perm[3] = -1                                   # a row that is not kept
    groups = None
    if paged:
        # rows 8..23 fill page 2 in order, rows 24..29 start page 4; every
        # other row is a run of its own
        perm[8:24] = torch.arange(32, 48, device=DEV)
        perm[24:30] = torch.arange(64, 70, device=DEV)
        taken = set(range(32, 48)) | set(range(64, 70))
        free = [s for s in range(nb * BS) if s not in taken]
        for i, r in enumerate([r for r in range(T) if not 8 <= r < 30]):
            perm[r] = free[(7 * i) % len(free)] if r != 3 else -1
        groups = _i32([[8, 16], [24, 6]]
                      + [[r, 1] for r in range(T) if not 8 <= r < 30])
    outs = []
    for impl in (ops, torch_ref):
        q = torch.zeros(T, nq, dtype=dtype, device=DEV)
        kc = torch.zeros(nb, G, BS, D, dtype=dtype, device=DEV)
        vc = torch.zeros(nb, G, VW, BS, dtype=dtype, device=DEV)
        args = (q, qkv.clone(), nq, nk, qw, kw, D, 0.25, 16, pos, v_first,
                lam if mix else None, kc, vc, perm, 1e-5)
        if impl is ops:
            ops.head_norm_store(*args, page_groups=groups)
        else:
            torch_ref.head_norm_store(*args)
        outs.append((q, kc, vc))
    tol = 0.04 if dtype == torch.bfloat16 else 1e-4
    for a, b in zip(*outs):
        assert (a.float() - b.float()).abs().max() <= tol


@pytest.mark.parametrize("sigmoid", [True, False])
@pytest.mark.parametrize("E,G,keep,gtop,top", [
    (8, 2, 1, 2, 3), (16, 1, 1, 1, 4), (12, 4, 2, 1, 5), (64, 8, 4, 2, 8),
    (6, 6, 4, 2, 2), (130, 10, 7, 3, 9)])
def test_route_topk(sigmoid, E, G, keep, gtop, top):
    T = 57
    logits = _rand(T, E + 3, std=2.0)
    corr = _rand(E, std=0.5, seed=4) - 0.4         # negative choice scores too
    for c, renorm in ((corr, True), (None, False)):
        ex = torch.zeros(T, top, dtype=torch.int32, device=DEV)
        wt = torch.zeros(T, top, device=DEV)
        rex, rwt = torch.zeros_like(ex), torch.zeros_like(wt)
        ops.route_topk(ex, wt, logits, c, E, G, keep, gtop, sigmoid, renorm,
                       1.7)
        torch_ref.route_topk(rex, rwt, logits, c, E, G, keep, gtop, sigmoid,
                             renorm, 1.7)
        assert torch.equal(ex.sort(-1)[0], rex.sort(-1)[0])
        o, ro = ex.argsort(-1), rex.argsort(-1)
        torch.testing.assert_close(wt.gather(1, o), rwt.gather(1, ro),
                                   rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 7])
@pytest.mark.parametrize("C,col0,big", [(300, 17, 1), (304, 16, 1),
                                        (2056, 8, 1), (2056, 8, 500)])
def test_causal_conv_silu(dtype, taps, C, col0, big):
    """(2056, 8) with the long portion: the 16-byte row-blocked kernel in
    bf16 (2, 3 or 4 taps); the others one lane per (row, channel)."""
    ld = C + col0 + 16
    news, hists, slots = ([9, 1, 1, 2, 30 * big, 1], [0, 5, 0, 1, 2, 1],
                          [3, 0, 5, 1, 2, 4])
    view = _ragged(news, hists, slots)
    T = sum(news)
    src = _rand(T, ld, dtype=dtype)
    w, b = _rand(C, taps, std=0.5, seed=1), _rand(C, seed=2)
    st0 = _rand(7, max(taps - 1, 1), C, dtype=dtype, seed=3)[:, :taps - 1]
    st0 = st0.contiguous()
    res = []
    for impl in (ops, torch_ref):
        out = torch.zeros(T, C, dtype=dtype, device=DEV)
        st = st0.clone()
        if impl is ops:
            ops.causal_conv_silu(out, src, col0, w, b, st, *view)
        else:
            torch_ref.causal_conv_silu(out, src, col0, w, b, st, view[0],
                                       view[1], view[2], view[4])
        res.append((out, st))
    got, ref = res[0][0].float(), res[1][0].float()
    if dtype == torch.bfloat16:     # one bf16 step of the value at most
        assert ((got - ref).abs() <= 0.008 * ref.abs() + 0.004).all()
    else:
        assert (got - ref).abs().max() <= 1e-5
    assert torch.equal(res[0][1], res[1][1])        # inputs are copied as is
    assert torch.equal(res[0][1][6], st0[6])        # an unused slot is untouched


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,G,N,P", [
    (4, 2, 32, 40), (3, 3, 64, 32), (3, 1, 24, 20), (2, 2, 128, 64),
    (2, 1, 200, 8), (5, 5, 16, 100), (2, 2, 256, 16), (6, 3, 7, 3),
    (2, 1, 64, 128), (3, 3, 24, 40), (2, 2, 8, 8), (2, 1, 128, 24),
    (2, 1, 400, 8), (1, 1, 512, 16)])
@pytest.mark.parametrize("stepped", [True, False])
@pytest.mark.parametrize("off", [3, 8])
def test_state_scan(dtype, H, G, N, P, stepped, off):
    """off = 8 with sizes that are multiples of 8 takes the 16-byte staging
    kernel in bf16; everything else the plain one."""
    news, hists, slots = [21, 1, 1, 2, 40], [0, 5, 0, 1, 2], [3, 0, 5, 1, 2]
    sf, sr, ss, _, pos = _ragged(news, hists, slots)
    T = sum(news)
    cx, cb, cc, cdt = off, off + H * P, off + H * P + G * N, off + H * P + 2 * G * N
    src = _rand(T, (cdt + H + 9) // 8 * 8, dtype=dtype, std=0.7)
    st0 = _rand(7, H, N, P, seed=5)
    if stepped:
        extra = (src, cdt, H, G, N, P, False, _rand(H, seed=6) - 1,
                 _rand(H, std=0.5, seed=7), _rand(H, seed=8), None)
    else:
        decay = torch.linspace(0.5, 0.999, H, device=DEV)
        extra = (None, 0, H, G, N, P, True, None, None, None, decay)
    def run(impl, **kw):
        y = torch.zeros(T, H * P, device=DEV)
        st = st0.clone()
        impl.state_scan(y, src, cx, cb, cc, *extra, st, sf, sr, ss, pos, **kw)
        return y, st

    ry, rst = run(torch_ref)
    scale = ry.abs().max().clamp(min=1.0)
    sscale = rst.abs().max().clamp(min=1.0)
    # the scan kernels, and the decode step kernel on the same ragged batch
    for kw in ({}, {"single": True}):
        y, st = run(ops, **kw)
        assert (y - ry).abs().max() <= 2e-4 * scale, kw
        assert (st - rst).abs().max() <= 2e-4 * sscale, kw
        assert torch.equal(st[6], st0[6])


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("C,groups,col", [(128, 2, 4), (96, 1, 4), (300, 3, 4),
                                          (2048, 8, 4), (2048, 8, 8),
                                          (6000, 2, 16), (1000, 5, 0),
                                          (20000, 4, 8)])
def test_gated_group_norm(out_dtype, C, groups, col):
    """Gate columns at multiples of 4 elements take the one-pass kernel in
    bf16 (parts up to 4096 channels)."""
    T = 11
    y = _rand(T, C, std=3.0)
    gsrc = _rand(T, C + 24, dtype=out_dtype, seed=2)
    gate = gsrc[:, col:col + C]
    w = _rand(C, seed=3)
    for first in (True, False):
        o = torch.zeros(T, C, dtype=out_dtype, device=DEV)
        r = torch.zeros_like(o)
        ops.gated_group_norm(o, y, gate, w, groups, 1e-5, first)
        torch_ref.gated_group_norm(r, y, gate, w, groups, 1e-5, first)
        tol = 0.05 if out_dtype == torch.bfloat16 else 1e-4
        assert (o.float() - r.float()).abs().max() <= tol


@pytest.mark.parametrize("dtype,exact", [(torch.bfloat16, False),
                                         (torch.bfloat16, True),
                                         (torch.float32, True)])
def test_paged_attention_distance_slopes(dtype, exact):
    H, G, D, VW, BS, nb = 6, 3, 64, 32, 16, 40
    news, hists = [70, 1, 5, 1], [0, 130, 60, 0]
    starts = [0, 70, 71, 76]
    T = sum(news)
    _, _, _, row_seq, pos = _ragged(news, hists, [0] * 4)
    kc = _rand(nb, G, BS, D, dtype=dtype)
    vc = _rand(nb, G, VW, BS, dtype=dtype, seed=1)
    q = _rand(T, H, D, dtype=dtype, seed=2)
    bt = torch.stack([torch.randperm(nb)[:10] for _ in news]).int().to(DEV)
    slopes = torch.tensor([2.0 ** (-8.0 * (h + 1) / H) for h in range(H)],
                          device=DEV)
    tiles = ops.build_attn_tiles(starts, hists, news, H, G, 1, DEV)
    for window in (0, 50):
        out = torch.zeros(T, H, VW, dtype=dtype, device=DEV)
        ref = torch.zeros_like(out)
        ops.paged_attention(out, q, kc, vc, bt, row_seq, pos, 0.125,
                            window=window, tiles=tiles, exact=exact,
                            max_ctx=131, slopes=slopes)
        torch_ref.paged_attention(ref, q, kc, vc, bt, row_seq, pos, 0.125,
                                  window=window, slopes=slopes)
        tol = 0.03 if dtype == torch.bfloat16 else 1e-4
        assert (out.float() - ref.float()).abs().max() <= tol
