"""The HIP kernels added for the Makezen mechanisms against their fp32
torch references (gpustack_amd/ops/torch_ref.py): per-head norm + rotation
row kernel, gated delta rule scan and step kernels, centred sandwich norms,
score cap and strided views of paged attention, SiLU-gated head norms, dual
RMS mix, head gates."""
import pytest
import torch

from gpustack_amd import ops
from gpustack_amd.ops import torch_ref

pytestmark = pytest.mark.gpu

DT = [torch.float32, torch.bfloat16]


def close(a, b, dtype, what=""):
    tol = 2e-5 if dtype == torch.float32 else 2e-2
    a, b = a.float().cpu(), b.float().cpu()
    scale = b.abs().max().clamp(min=1.0)
    assert (a - b).abs().max() / scale < tol, what


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("W", [22, 64, 1500, 5000])
def test_centred_sandwich(dtype, W):
    g = torch.Generator().manual_seed(W)
    T, eps = 7, 1e-5
    x = torch.randn(T, W, generator=g) * 2 + 1
    a = (torch.randn(T, W, generator=g) - 3).to(dtype)
    pw, nw = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    for center in (True, False):
        xr, hr = x.clone(), torch.zeros(T, W, dtype=dtype)
        torch_ref.sandwich_add_norm(xr, a, pw, 0.7, eps, None, nw, hr, center)
        xg, hg = x.cuda(), torch.zeros(T, W, dtype=dtype, device="cuda")
        ops.sandwich_add_norm(xg, a.cuda(), pw.cuda(), 0.7, eps, None,
                              nw.cuda(), hg, center=center)
        close(xg, xr, torch.float32)
        close(hg, hr, dtype)
    # the opening half alone (fp32 rows in, a norm out)
    hr = torch.zeros(T, W, dtype=dtype)
    torch_ref.sandwich_add_norm(x.clone(), None, None, 0.0, eps, None, nw, hr,
                                True)
    hg = torch.zeros(T, W, dtype=dtype, device="cuda")
    ops.sandwich_add_norm(x.cuda(), None, None, 0.0, eps, None, nw.cuda(), hg,
                          center=True)
    close(hg, hr, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("half_layout", [True, False])
@pytest.mark.parametrize("shape", [
    # q heads, k heads, dim, value size, normed, rot0, rotated dims
    (3, 2, 10, 7, 10, 0, 6), (8, 2, 64, 48, 64, 0, 16), (5, 1, 33, 9, 20, 21, 12),
    (4, 4, 128, 128, 128, 0, 128)])
def test_head_rope_store(dtype, half_layout, shape):
    H, G, d, dv, nd, rot0, rd = shape
    g = torch.Generator().manual_seed(d)
    T, BS, eps = 37, 16, 1e-5
    src = (torch.randn(T, (H + G) * d + G * dv + 8, generator=g)).to(dtype)
    qw, kw = torch.rand(nd, generator=g) + 0.5, torch.rand(nd, generator=g) + 0.5
    invf = torch.rand(rd // 2, generator=g)
    pos = torch.randint(0, 3000, (T,), generator=g).to(torch.int32)
    slots = torch.randperm(5 * BS, generator=g)[:T]
    slots[3] = -1
    args = (0, H, d, None, nd, rot0, H * d, G, d, None, nd, rot0, (H + G) * d)

    def run(dev, page_groups=None):
        to = lambda t: t.to(dev)
        q = torch.zeros(T, H * d, dtype=dtype, device=dev)
        kc = torch.zeros(6, G, BS, d, dtype=dtype, device=dev)
        vc = torch.zeros(6, G, dv, BS, dtype=dtype, device=dev)
        a = list(args)
        a[3], a[9] = to(qw), to(kw)
        fn = ops.head_rope_store if dev == "cuda" else torch_ref.head_rope_store
        kw_ = {"page_groups": page_groups} if dev == "cuda" else {}
        fn(q, to(src), *a, to(invf), half_layout, 1.3, to(pos), kc, vc,
           to(slots), eps, **kw_)
        return q, kc, vc

    ref = run("cpu")
    for got in (run("cuda"),):
        for a, b, nm in zip(got, ref, "qkv"):
            close(a, b, dtype, nm)
    # values tied to the key head's first channels (a latent row)
    def run_tied(dev):
        to = lambda t: t.to(dev)
        q = torch.zeros(T, H * d, dtype=dtype, device=dev)
        kc = torch.zeros(6, G, BS, d, dtype=dtype, device=dev)
        vc = torch.zeros(6, G, min(dv, d), BS, dtype=dtype, device=dev)
        fn = ops.head_rope_store if dev == "cuda" else torch_ref.head_rope_store
        fn(q, to(src), 0, H, d, None, 0, -1, H * d, G, d, to(kw), nd, rot0, -1,
           to(invf), half_layout, 1.0, to(pos), kc, vc, to(slots), eps)
        return q, kc, vc

    for a, b, nm in zip(run_tied("cuda"), run_tied("cpu"), "qkv"):
        close(a, b, dtype, "tied " + nm)


@pytest.mark.parametrize("dtype", DT)
def test_head_rope_store_values_by_page(dtype):
    """Prompt rows: the values leave page by page, the rest row by row."""
    H, G, d, dv = 4, 2, 32, 16
    g = torch.Generator().manual_seed(1)
    BS, eps = 16, 1e-5
    starts, hists, news = [0, 40], [5, 0], [40, 21]
    T = 61
    src = torch.randn(T, (H + G) * d + G * dv, generator=g).to(dtype)
    w = torch.rand(d, generator=g) + 0.5
    invf = torch.rand(4, generator=g)
    pos = torch.tensor(list(range(5, 45)) + list(range(21)), dtype=torch.int32)
    slots = torch.cat([torch.arange(5, 45) + 16 * 2, torch.arange(21)]).long()
    groups = ops.build_page_groups(starts, hists, news, BS, "cuda")

    def run(dev, pg=None):
        to = lambda t: t.to(dev)
        q = torch.zeros(T, H * d, dtype=dtype, device=dev)
        kc = torch.zeros(6, G, BS, d, dtype=dtype, device=dev)
        vc = torch.zeros(6, G, dv, BS, dtype=dtype, device=dev)
        fn = ops.head_rope_store if dev == "cuda" else torch_ref.head_rope_store
        kw_ = {"page_groups": pg} if dev == "cuda" else {}
        fn(q, to(src), 0, H, d, to(w), d, 0, H * d, G, d, to(w), d, 0,
           (H + G) * d, to(invf), True, 1.0, to(pos), kc, vc, to(slots), eps,
           **kw_)
        return q, kc, vc

    ref = run("cpu")
    for a, b, nm in zip(run("cuda", groups), ref, "qkv"):
        close(a, b, dtype, nm)

    # a latent row: the values are the finished key row's first channels
    # and leave page by page out of the key pool
    QR, R, RD = 24, 48, 8
    src2 = torch.randn(T, QR + R + RD, generator=g).to(dtype)
    wq, wr = torch.rand(QR, generator=g) + 0.5, torch.rand(R, generator=g) + 0.5

    def run_latent(dev, pg=None):
        to = lambda t: t.to(dev)
        cq = torch.zeros(T, QR, dtype=dtype, device=dev)
        kc = torch.zeros(6, 1, BS, R + RD, dtype=dtype, device=dev)
        vc = torch.zeros(6, 1, R, BS, dtype=dtype, device=dev)
        fn = ops.head_rope_store if dev == "cuda" else torch_ref.head_rope_store
        kw_ = {"page_groups": pg} if dev == "cuda" else {}
        fn(cq, to(src2), 0, 1, QR, to(wq), QR, -1, QR, 1, R + RD, to(wr), R, R,
           -1, to(invf), True, 1.2, to(pos), kc, vc, to(slots), eps, **kw_)
        return cq, kc, vc

    ref = run_latent("cpu")
    for pg in (None, groups):
        for a, b, nm in zip(run_latent("cuda", pg), ref, "qkv"):
            close(a, b, dtype, "latent " + nm)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("H,G,N,P", [(4, 2, 6, 5), (2, 2, 16, 8), (3, 1, 5, 12),
                                     (4, 1, 64, 64), (2, 2, 128, 128),
                                     (6, 3, 40, 20), (1, 1, 200, 36)])
@pytest.mark.parametrize("single", [False, True])
def test_delta_scan(dtype, H, G, N, P, single):
    """Prompt portions and single rows, fresh and continued states, slots
    out of order; `single` takes the step kernel where the sizes allow."""
    g = torch.Generator().manual_seed(N + P)
    nqk = G * N
    if single:
        news, hists = [1, 1, 1], [0, 7, 300]
    else:
        news, hists = [19, 1, 40], [0, 5, 33]
    T, nseq = sum(news), len(news)
    # sizes of a multiple of 8 sit at columns of a multiple of 8 in rows of
    # a multiple of 8, which is what the 16-byte staging kernel asks for
    off = 8 if N % 8 == 0 and P % 8 == 0 else 1
    width = off + 2 * nqk + H * P + 3
    src = torch.randn(T, width + (-width) % 8, generator=g).to(dtype)
    gates = (torch.randn(T, 2 * H + 2, generator=g) * 2).to(dtype)
    dt_bias = torch.randn(H, generator=g)
    a_log = torch.randn(H, generator=g) - 1
    state0 = torch.randn(5, H, N, P, generator=g)
    meta = lambda a: torch.tensor(a, dtype=torch.int32)
    first = [sum(news[:i]) for i in range(nseq)]
    pos = meta([h + j for h, n in zip(hists, news) for j in range(n)])
    slots = meta([3, 0, 4])

    def run(dev):
        to = lambda t: t.to(dev)
        y = torch.zeros(T, H * P, device=dev)
        st = state0.clone().to(dev)
        fn = ops.delta_scan if dev == "cuda" else torch_ref.delta_scan
        kw_ = {"single": single} if dev == "cuda" else {}
        fn(y, to(src), off, off + nqk, off + 2 * nqk, to(gates), 1, 1 + H, H,
           G, N, P, to(dt_bias), to(a_log), st, to(meta(first)), to(meta(news)),
           to(slots), to(pos), **kw_)
        return y, st

    (yr, sr), (yg, sg) = run("cpu"), run("cuda")
    tol = 1e-4
    assert (yg.cpu() - yr).abs().max() / yr.abs().max().clamp(min=1) < tol
    assert (sg.cpu() - sr).abs().max() / sr.abs().max().clamp(min=1) < tol
    # untouched slots stay what they were
    assert torch.equal(sg.cpu()[[1, 2]], state0[[1, 2]])


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("mode", [0, 1, 2])
@pytest.mark.parametrize("C,groups", [(24, 4), (256, 4), (100, 1)])
def test_gated_group_norm_modes(dtype, mode, C, groups):
    g = torch.Generator().manual_seed(C)
    T = 9
    y = torch.randn(T, C, generator=g)
    u = torch.randn(T, C + 16, generator=g).to(dtype)
    w = torch.rand(C, generator=g) + 0.5
    ref = torch.zeros(T, C, dtype=dtype)
    torch_ref.gated_group_norm(ref, y, u[:, 8:8 + C], w, groups, 1e-5, mode)
    got = torch.zeros(T, C, dtype=dtype, device="cuda")
    ops.gated_group_norm(got, y.cuda(), u.cuda()[:, 8:8 + C], w.cuda(), groups,
                         1e-5, mode)
    close(got, ref, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("W", [18, 192, 3000])
def test_dual_rms_mix(dtype, W):
    g = torch.Generator().manual_seed(W)
    T = 6
    a, b = (torch.randn(T, W, generator=g) * 3).to(dtype), \
        torch.randn(T, W, generator=g).to(dtype)
    wa, wb = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    ref = torch.zeros(T, W, dtype=dtype)
    torch_ref.dual_rms_mix(ref, a, wa, b, wb, 1e-5)
    got = torch.zeros(T, W, dtype=dtype, device="cuda")
    ops.dual_rms_mix(got, a.cuda(), wa.cuda(), b.cuda(), wb.cuda(), 1e-5)
    close(got, ref, dtype)


@pytest.mark.parametrize("dtype", DT)
def test_head_gate(dtype):
    g = torch.Generator().manual_seed(0)
    H, T, VD = 5, 11, 7
    o = torch.randn(H, T, VD, generator=g).to(dtype)
    u = torch.randn(T, 40, generator=g).to(dtype)
    ref = torch.zeros(T, H * VD, dtype=dtype)
    torch_ref.head_gate(ref, o, u, 33)
    got = torch.zeros(T, H * VD, dtype=dtype, device="cuda")
    ops.head_gate(got, o.cuda(), u.cuda(), 33)
    close(got, ref, dtype)


@pytest.mark.parametrize("dtype", DT)
@pytest.mark.parametrize("exact", [False, True])
@pytest.mark.parametrize("D,VW", [(64, 32), (448, 384)])
def test_paged_attention_cap_window_sink_on_strided_views(dtype, exact, D, VW):
    """Multi-query attention on head-major q / out buffers handed over as
    [T, heads, *] views, with a window, sinks and a score cap; also at a
    latent row's sizes (value channels beyond 256)."""
    g = torch.Generator().manual_seed(5)
    H, BS = 6, 16
    starts, hists, news = [0, 30], [50, 0], [30, 9]
    T = 39
    nb = 8
    kc = torch.randn(nb, 1, BS, D, generator=g).to(dtype)
    vc = torch.randn(nb, 1, VW, BS, generator=g).to(dtype)
    q_hts = (torch.randn(H, T, D, generator=g) * (64.0 / D) ** 0.5).to(dtype)
    bt = torch.tensor([[2, 5, 1, 7, 3], [4, 0, 6, 0, 0]], dtype=torch.int32)
    row_seq = torch.tensor([0] * 30 + [1] * 9, dtype=torch.int32)
    pos = torch.tensor(list(range(50, 80)) + list(range(9)), dtype=torch.int32)
    sinks = torch.randn(H, generator=g)
    for window, cap in ((0, 0.0), (21, 0.0), (0, 1.5), (33, 2.5)):
        ref = torch.zeros(H, T, VW, dtype=dtype)
        torch_ref.paged_attention(ref.transpose(0, 1), q_hts.transpose(0, 1),
                                  kc, vc, bt, row_seq, pos, 0.2, window=window,
                                  sinks=sinks, softcap=cap)
        got = torch.zeros(H, T, VW, dtype=dtype, device="cuda")
        tiles = ops.build_attn_tiles(starts, hists, news, H, 1, 1, "cuda")
        ops.paged_attention(got.transpose(0, 1), q_hts.cuda().transpose(0, 1),
                            kc.cuda(), vc.cuda(), bt.cuda(), row_seq.cuda(),
                            pos.cuda(), 0.2, window=window, sinks=sinks.cuda(),
                            tiles=tiles, exact=exact, max_ctx=80, softcap=cap)
        close(got, ref, dtype, (window, cap))
