"""Each hand-written kernel alone against a plain float64 reference, at sizes other than the
tiny models': head sizes 16..1024, odd head counts and groups, widths and vocabularies that are
no power of two, ragged row counts."""
import math

import numpy as np
import pytest
import torch

from plain import llama_plain as P
from plain import sampler_plain as SP

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
PAGE = 64


def K():
    from picolm_amd import kernels
    return kernels


def tol(dtype, scale):
    return (2e-2 if dtype == torch.bfloat16 else 2e-5) * scale + (1e-3 if dtype == torch.bfloat16 else 1e-6)


# ------------------------------------------------------------------------------------------ rows
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D,V", [(1, 80, 131), (37, 4096, 500)])
def test_embed(dtype, T, D, V):
    g = torch.Generator().manual_seed(0)
    table = torch.randn(V, D, generator=g).to(dtype).to(DEV)
    tokens = torch.randint(0, V, (T,), generator=g, dtype=torch.int32).to(DEV)
    out = torch.empty(T, D, device=DEV)
    K().embed(table, tokens, out)
    assert torch.equal(out, table.float()[tokens.long()])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,D,eps", [(1, 80, 1e-5), (19, 4096, 1e-6), (5, 1000, 1e-2)])
def test_rmsnorm(out_dtype, T, D, eps):
    g = torch.Generator().manual_seed(1)
    x = (torch.randn(T, D, generator=g) * 3).to(DEV)
    w = (1 + 0.3 * torch.randn(D, generator=g)).to(DEV)
    out = torch.empty(T, D, dtype=out_dtype, device=DEV)
    K().rmsnorm(x, w, eps, out)
    ref = P.rmsnorm(x.cpu().numpy(), w.cpu().numpy(), eps)
    err = np.abs(out.double().cpu().numpy() - ref).max()
    assert err <= tol(out_dtype, np.abs(ref).max())
    # selected rows
    rows = torch.tensor([T - 1, 0], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, D, dtype=out_dtype, device=DEV)
    K().rmsnorm(x, w, eps, out2, rows)
    assert torch.equal(out2[0], out[T - 1]) and torch.equal(out2[1], out[0])


# ------------------------------------------------------------------------------------------ gemm
def gemm_ref(a, w, epi, c0):
    y = a.double().cpu() @ w.double().cpu().T
    if epi == 1:
        return c0.double().cpu() + y
    if epi == 2:
        g_, u = y[:, 0::2], y[:, 1::2]
        return g_ / (1 + torch.exp(-g_)) * u
    return y


def run_gemm(fn, M, N, Kd, epi, adt, wdt, cdt, **kw):
    g = torch.Generator().manual_seed(M * 7 + N)
    a = torch.randn(M, Kd, generator=g).to(adt).to(DEV)
    w = (torch.randn(N, Kd, generator=g) * 0.1).to(wdt).to(DEV)
    c = torch.randn(M, N // 2 if epi == 2 else N, generator=g).to(cdt).to(DEV)
    c0 = c.clone()
    fn(a, w, c, epi, **kw)
    ref = gemm_ref(a, w, epi, c0)
    err = (c.double().cpu() - ref).abs().max().item()
    assert err <= tol(cdt, ref.abs().max().item()), (M, N, Kd, epi, err)


@pytest.mark.parametrize("M", [1, 3, 17, 64, 65, 200])
@pytest.mark.parametrize("N,Kd", [(6, 5), (130, 77), (352, 176)])
def test_gemm_generic_f32(M, N, Kd):
    for epi in (0, 1, 2):
        run_gemm(K().gemm_generic, M, N, Kd, epi, torch.float32, torch.float32, torch.float32)


def test_gemm_generic_mixed_types():
    for adt, wdt, cdt in [(torch.bfloat16, torch.float32, torch.float32), (torch.float32, torch.bfloat16, torch.bfloat16),
                          (torch.bfloat16, torch.bfloat16, torch.bfloat16)]:
        for epi in (0, 2):
            run_gemm(K().gemm_generic, 9, 70, 45, epi, adt, wdt, cdt)
    run_gemm(K().gemm_generic, 9, 70, 45, 1, torch.bfloat16, torch.float32, torch.float32)


@pytest.mark.parametrize("M", [1, 2, 15, 16, 17, 33, 64])
@pytest.mark.parametrize("N,Kd", [(96, 64), (130, 264), (1000, 1000), (4096, 1024)])
def test_gemm_skinny(M, N, Kd):
    for epi, cdt in ((0, torch.float32), (0, torch.bfloat16), (1, torch.float32), (2, torch.bfloat16)):
        run_gemm(K().gemm_skinny, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt)


@pytest.mark.parametrize("M", [1, 5, 8, 9, 16])
@pytest.mark.parametrize("N,Kd", [(100, 128), (16, 64), (4096, 4096), (6144, 1024), (8192, 576), (10240, 512), (4090, 14336)])
def test_gemm_skinny_through_stages_of_a_waves_own(M, N, Kd):
    """One round of workgroups of 16, 24, 32 or 40 weight rows with K in multiples of 64: weights
    and activations go through LDS stages of each wave (three to eight of them, by the rows of both).
    Few slices of K (some waves have none), many (a wave goes round its stages several times), a
    last workgroup with fewer rows than the others; and the older kernel must give the same sums."""
    for epi, cdt in ((0, torch.float32), (0, torch.bfloat16), (1, torch.float32), (2, torch.bfloat16)):
        run_gemm(K().gemm_skinny, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt)
    g = torch.Generator().manual_seed(N + M)
    a = torch.randn(M, Kd, generator=g).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, Kd, generator=g) * 0.1).to(torch.bfloat16).to(DEV)
    c1, c2 = torch.zeros(M, N, device=DEV), torch.zeros(M, N, device=DEV)
    K().gemm_skinny(a, w, c1, 0)
    K().gemm_skinny(a, w, c2, 0, variant=9)          # never staged
    assert (c1 - c2).abs().max().item() <= 1e-5 * c2.abs().max().item()


@pytest.mark.parametrize("variant", [1, 2, 3, 4, 5, 6])
def test_gemm_skinny_variants(variant):
    M = {1: 16, 2: 13, 3: 32, 4: 21, 5: 64, 6: 50}[variant]
    for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
        run_gemm(K().gemm_skinny, M, 530, 1032, epi, torch.bfloat16, torch.bfloat16, cdt, variant=variant)


@pytest.mark.parametrize("M", [65, 128, 300, 1111])
@pytest.mark.parametrize("N,Kd", [(96, 64), (130, 264), (1000, 1000), (512, 2048)])
def test_gemm_tiled(M, N, Kd):
    for epi, cdt in ((0, torch.float32), (0, torch.bfloat16), (1, torch.float32), (2, torch.bfloat16)):
        run_gemm(K().gemm_tiled, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt)


@pytest.mark.parametrize("variant,splits", [(12, 2), (12, 8), (13, 4), (11, 4), (9, 3)])
def test_gemm_tiled_split_along_k(variant, splits):
    """K cut into parts whose partial sums a second kernel adds in order: every epilogue, ragged
    M and N, and the same bits on every run."""
    for M, N, Kd in ((64, 4096 + 8, 64 * splits * 3), (17, 132, 64 * splits), (300, 260, 64 * splits * 2)):
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32), (0, torch.bfloat16)):
            run_gemm(lambda a, w, c, e: K().gemm_tiled_splitk(a, w, c, e, variant, splits), M, N, Kd, epi,
                     torch.bfloat16, torch.bfloat16, cdt)
    a = torch.randn(64, 64 * splits * 5, device=DEV).to(torch.bfloat16)
    w = torch.randn(4096, 64 * splits * 5, device=DEV).to(torch.bfloat16)
    outs = []
    for _ in range(3):
        c = torch.zeros(64, 4096, device=DEV)
        K().gemm_tiled_splitk(a, w, c, 0, variant, splits)
        outs.append(c)
    assert torch.equal(outs[0], outs[1]) and torch.equal(outs[0], outs[2])
    with pytest.raises(Exception, match="multiple"):
        K().gemm_tiled_splitk(a[:, :64 * splits + 64].contiguous(), w[:, :64 * splits + 64].contiguous(), outs[0], 0, variant, splits)


def test_gemm_medium_batches_pick_their_splits():
    from picolm_amd.kernels import medium_gemm_splits
    assert medium_gemm_splits(64, 28672, 4096) == 1          # enough tiles of its own
    assert medium_gemm_splits(64, 6144, 4096) == 4
    assert medium_gemm_splits(64, 4096, 4096) == 8
    assert medium_gemm_splits(64, 4096, 14336) == 8
    assert medium_gemm_splits(64, 4096, 64 * 3) == 1         # K does not split evenly
    assert medium_gemm_splits(33, 130, 4096) == 1            # N no multiple of 4
    # never a few more workgroups than CUs: 80 tiles in two parts, 160 tiles uncut, 40 tiles in four
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    for N in (10240, 20480, 5120):
        assert (N // 128) * medium_gemm_splits(32, N, 8192) <= cus < 2 * (N // 128) * medium_gemm_splits(32, N, 8192)


def test_decode_attention_picks_eight_waves_up_to_two_workgroups_a_cu():
    waves = K().lib().picolm_attn_decode_mfma_waves
    assert waves(8, 32, 8) == 8 and waves(64, 32, 8) == 8            # 64 and 512 workgroups
    assert waves(65, 32, 8) == 4 and waves(16, 32, 32) == 8 and waves(17, 32, 32) == 4
    assert waves(4, 128, 2) == 8 and waves(512, 128, 2) == 4         # 64 heads a group: two workgroups each
    for M, N, Kd in ((64, 4096, 4096), (40, 6144, 1024), (17, 260, 192), (64, 28672 // 4, 512), (8, 16384 + 2, 128),
                     (5, 128 * 256, 64)):
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
            run_gemm(K().gemm, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt)


def test_gemm_of_a_short_prompt_is_cut_along_k():
    """More than 64 rows but tiles for half of the CUs or fewer (a short prompt's products into
    the model's width): the tiled product is cut along K like a wide decode batch's.  Every
    epilogue against the plain product, with and without the cut (N no multiple of 1024: uncut)."""
    k = K()
    ws = k.SPLITK_WS_FLOATS
    assert k.lib().picolm_gemm_tiled_norm_parts(512, 4096, 4096, k.c_int64(ws)) == 4           # cut: N / 1024
    assert k.lib().picolm_gemm_tiled_norm_parts(512, 4096, 4096, k.c_int64(0)) == 32          # no room: per column of tiles
    assert k.lib().picolm_gemm_tiled_norm_parts(2048, 4096, 4096, k.c_int64(ws)) == 16        # enough tiles
    for M, N, Kd in ((512, 4096, 4096), (300, 1024, 512), (65, 2048, 14336 // 7), (512, 4096 + 8, 1024), (200, 2048, 64 * 3)):
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32), (0, torch.bfloat16)):
            run_gemm(k.gemm, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt)


@pytest.mark.parametrize("M", [1, 8, 16])
@pytest.mark.parametrize("D", [48, 256, 4096, 8192])
def test_gemm_with_a_norm_split_between_two_products(M, D):
    """The product that finishes rows of the residual stream prepares the RMSNorm that follows
    (bf16(x * w) and partial sums of x^2), the next product applies 1 / sqrt(mean(x^2) + eps) to
    its sums: together they must give norm-then-product.  Rows of very different size, so that a
    factor taken from the wrong row shows; every kernel that can be the consumer.  (A width of
    8,192 makes two rounds of 16-row workgroups: the producer then takes 32 rows a workgroup.)"""
    g = torch.Generator().manual_seed(M * 31 + D)
    eps, K1 = 1e-5, 192
    x0 = torch.randn(M, D, generator=g) * (10.0 ** torch.arange(M).remainder(5).sub(2).float())[:, None]
    a1 = torch.randn(M, K1, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(D, K1, generator=g) * 0.05).to(torch.bfloat16)
    nw = 1.0 + 0.3 * torch.randn(D, generator=g)
    x = x0.clone().to(DEV)
    h = torch.full((M, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ssq = torch.full((K().linked_norm_parts(M, D, K1), 16), float("nan"), device=DEV)
    K().gemm_linked(a1.to(DEV), w1.to(DEV), x, 1, prepare=(nw.to(DEV), h, ssq))
    x_ref = x0.double() + a1.double() @ w1.double().T
    assert (x.double().cpu() - x_ref).abs().max() <= tol(torch.float32, x_ref.abs().max().item()) + 1e-2 * 0
    assert torch.equal(h.cpu(), (x.cpu() * nw).to(torch.bfloat16))          # from the very values it stored
    total = ssq[:, :M].double().sum(dim=0).cpu()
    want = (x.double().cpu() ** 2).sum(dim=1)
    assert ((total - want).abs() <= 1e-5 * want + 1e-30).all()
    normed = x.double().cpu() / torch.sqrt((x.double().cpu() ** 2).mean(dim=1, keepdim=True) + eps) * nw.double()
    if D % 8:
        return
    for N2 in (48, 16 * 300 - 6, 16384 + 32, 40000):
        if N2 > 20000 and D > 256:
            continue                        # (a large reference product on the CPU for nothing new)
        w2 = (torch.randn(N2, D, generator=g) * 0.1).to(torch.bfloat16)
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
            c = torch.randn(M, N2 // 2 if epi == 2 else N2, generator=g).to(cdt).to(DEV)
            ref = gemm_ref(normed, w2, epi, c.clone())
            K().gemm_linked(h, w2.to(DEV), c, epi, prepared=(ssq, D, eps))
            err = (c.double().cpu() - ref).abs().max().item()
            assert err <= tol(torch.bfloat16, ref.abs().max().item()), (M, D, N2, epi, err)


@pytest.mark.parametrize("M", [17, 40, 64])
@pytest.mark.parametrize("D", [1024, 3072])
def test_gemm_with_a_norm_split_between_two_products_of_a_wide_decode_batch(M, D):
    """17 to 64 rows: the kernel that adds the parts of a product cut along K prepares the norm,
    and the next product takes it in that same kernel (cut) or in the tile kernel (uncut)."""
    k = K()
    g = torch.Generator().manual_seed(M * 31 + D)
    eps, K1 = 1e-6, 512
    assert k.medium_gemm_splits(M, D, K1) > 1
    x0 = torch.randn(M, D, generator=g) * (10.0 ** torch.arange(M).remainder(5).sub(2).float())[:, None]
    a1 = torch.randn(M, K1, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(D, K1, generator=g) * 0.05).to(torch.bfloat16)
    nw = 1.0 + 0.3 * torch.randn(D, generator=g)
    assert k.gemm_links_norms(a1.to(DEV), w1.to(DEV), x0.to(DEV), 1, prepares=True)
    x = x0.clone().to(DEV)
    h = torch.full((M, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    ssq = torch.full((k.linked_norm_parts(M, D, K1), k.linked_norm_rows(M)), float("nan"), device=DEV)
    assert tuple(ssq.shape) == (D // 1024, 64)
    k.gemm_linked(a1.to(DEV), w1.to(DEV), x, 1, prepare=(nw.to(DEV), h, ssq))
    x_ref = x0.double() + a1.double() @ w1.double().T
    assert (x.double().cpu() - x_ref).abs().max() <= tol(torch.float32, x_ref.abs().max().item())
    assert torch.equal(h.cpu(), (x.cpu() * nw).to(torch.bfloat16))          # from the very values it stored
    total = ssq[:, :M].double().sum(dim=0).cpu()
    want = (x.double().cpu() ** 2).sum(dim=1)
    assert ((total - want).abs() <= 1e-5 * want + 1e-30).all()
    normed = x.double().cpu() / torch.sqrt((x.double().cpu() ** 2).mean(dim=1, keepdim=True) + eps) * nw.double()
    for N2 in (2048, 128 * 200 + 6):             # cut along K / enough tiles of its own
        w2 = (torch.randn(N2, D, generator=g) * 0.1).to(torch.bfloat16)
        assert (k.medium_gemm_splits(M, N2, D) > 1) == (N2 == 2048)
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
            c = torch.randn(M, N2 // 2 if epi == 2 else N2, generator=g).to(cdt).to(DEV)
            assert k.gemm_links_norms(h, w2.to(DEV), c, epi, prepares=False)
            ref = gemm_ref(normed, w2, epi, c.clone())
            k.gemm_linked(h, w2.to(DEV), c, epi, prepared=(ssq, D, eps))
            err = (c.double().cpu() - ref).abs().max().item()
            assert err <= tol(torch.bfloat16, ref.abs().max().item()), (M, D, N2, epi, err)
    # what the kernels cannot do is said, not done wrongly
    w3 = torch.zeros(1000, D, dtype=torch.bfloat16, device=DEV)          # cut, and N no multiple of 1024
    c3 = torch.zeros(M, 1000, device=DEV)
    assert k.medium_gemm_splits(M, 1000, D) > 1 and not k.gemm_links_norms(h, w3, c3, 0, prepares=False)
    with pytest.raises(k.KernelError):
        k.gemm_linked(h, w3, c3, 0, prepared=(ssq, D, eps))
    assert not k.gemm_links_norms(h, torch.zeros(128 * 200, D, dtype=torch.bfloat16, device=DEV),
                                  torch.zeros(M, 128 * 200, device=DEV), 1, prepares=True)     # uncut: no preparing


@pytest.mark.parametrize("M,D", [(65, 1024), (300, 1024), (2048, 1024), (65, 4352), (300, 4352), (2048, 10240), (1536, 6144)])
def test_gemm_with_a_norm_split_between_two_products_of_a_prefill_step(M, D):
    """More than 64 rows: the tile kernels keep sums for every row, one share per column of tiles;
    10240 columns at 2048 rows are two launches with different tiles, which must meet without a seam;
    6144 columns at 1536 or 2048 rows take the tiles of 192 columns, in either role."""
    k = K()
    g = torch.Generator().manual_seed(M * 31 + D)
    eps, K1 = 1e-5, 256
    x0 = torch.randn(M, D, generator=g) * (10.0 ** torch.arange(M).remainder(5).sub(2).float())[:, None]
    a1 = torch.randn(M, K1, generator=g).to(torch.bfloat16)
    w1 = (torch.randn(D, K1, generator=g) * 0.05).to(torch.bfloat16)
    nw = 1.0 + 0.3 * torch.randn(D, generator=g)
    x = x0.clone().to(DEV)
    assert k.gemm_links_norms(a1.to(DEV), w1.to(DEV), x, 1, prepares=True)
    h = torch.full((M, D), float("nan"), dtype=torch.bfloat16, device=DEV)
    parts, rows = k.linked_norm_parts(M, D, K1), k.linked_norm_rows(M)
    assert parts > 0 and rows >= M and rows % 64 == 0
    ssq = torch.full((parts, rows), float("nan"), device=DEV)
    k.gemm_linked(a1.to(DEV), w1.to(DEV), x, 1, prepare=(nw.to(DEV), h, ssq))
    x_ref = x0.double() + a1.double() @ w1.double().T
    assert (x.double().cpu() - x_ref).abs().max() <= tol(torch.float32, x_ref.abs().max().item())
    assert torch.equal(h.cpu(), (x.cpu() * nw).to(torch.bfloat16))          # from the very values it stored
    total = ssq[:, :M].double().sum(dim=0).cpu()
    want = (x.double().cpu() ** 2).sum(dim=1)
    assert ((total - want).abs() <= 1e-5 * want + 1e-30).all()
    normed = x.double().cpu() / torch.sqrt((x.double().cpu() ** 2).mean(dim=1, keepdim=True) + eps) * nw.double()
    for N2 in (384, 3072 + 6) + ((6144,) if (M, D) == (2048, 1024) else ()):
        w2 = (torch.randn(N2, D, generator=g) * 0.1).to(torch.bfloat16)
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
            c = torch.randn(M, N2 // 2 if epi == 2 else N2, generator=g).to(cdt).to(DEV)
            assert k.gemm_links_norms(h, w2.to(DEV), c, epi, prepares=False)
            ref = gemm_ref(normed, w2, epi, c.clone())
            k.gemm_linked(h, w2.to(DEV), c, epi, prepared=(ssq, D, eps))
            err = (c.double().cpu() - ref).abs().max().item()
            assert err <= tol(torch.bfloat16, ref.abs().max().item()), (M, D, N2, epi, err)
    # K no multiple of 64: the older tiles, which take no part
    assert not k.gemm_links_norms(torch.zeros(M, 72, dtype=torch.bfloat16, device=DEV),
                                  torch.zeros(D, 72, dtype=torch.bfloat16, device=DEV), x, 1, prepares=True)
    # the answer beforehand and the kernels' own conditions agree at widths that some of them refuse
    # (an odd one: the tiles write pairs of columns; cut along K, one that is no multiple of 1024):
    # a yes runs, and an odd width gets a no
    for width in (515, 1500, 1032):
        a, w = torch.zeros(M, 512, dtype=torch.bfloat16, device=DEV), torch.zeros(width, 512, dtype=torch.bfloat16, device=DEV)
        c = torch.zeros(M, width, device=DEV)
        yes = k.gemm_links_norms(a, w, c, 1, prepares=True)
        assert yes == (k.linked_norm_parts(M, width, 512) > 0) and not (yes and width % 2)
        if yes:
            k.gemm_linked(a, w, c, 1, prepare=(torch.ones(width, device=DEV), torch.empty(M, width, dtype=torch.bfloat16, device=DEV),
                                               torch.empty(k.linked_norm_parts(M, width, 512), k.linked_norm_rows(M), device=DEV)))


def test_gemm_tiles_of_192_and_320_columns_where_they_fill_the_rounds_better():
    """1536 rows of 6144 columns: 144 tiles of 256 x 256 or 192 of 192 columns; 2048 rows of 10240
    columns: 320 tiles or 256 of 320 columns; the plan takes the latter in both cases (the wide
    tile not with the adding epilogue)."""
    for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
        run_gemm(K().gemm_tiled, 1536, 6144, 128, epi, torch.bfloat16, torch.bfloat16, cdt)
        run_gemm(K().gemm_tiled, 1500, 6144, 64, epi, torch.bfloat16, torch.bfloat16, cdt)
        run_gemm(K().gemm_tiled, 2048, 10240, 128, epi, torch.bfloat16, torch.bfloat16, cdt)
        run_gemm(K().gemm_tiled, 2000, 10240, 64, epi, torch.bfloat16, torch.bfloat16, cdt)


def test_gemm_tiled_splits_a_partial_last_round():
    """300 tiles of 256x256 on 256 CUs: the columns past the first 256 tiles take the half-height
    tile in a launch of their own; the seam must not show in any epilogue."""
    for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
        run_gemm(K().gemm_tiled, 512, 150 * 256 - 10, 64, epi, torch.bfloat16, torch.bfloat16, cdt)
        run_gemm(K().gemm_tiled, 300, 150 * 256 - 10, 128, epi, torch.bfloat16, torch.bfloat16, cdt)


@pytest.mark.parametrize("variant", [1, 4])
def test_gemm_tiled_block_tiles(variant):
    for M, N, Kd in ((300, 530, 1032), (70, 260, 72), (513, 100, 200), (9, 700, 136), (64, 130, 64)):
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32)):
            run_gemm(K().gemm_tiled, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt, variant=variant)


@pytest.mark.parametrize("variant", [9, 10, 11, 12, 13, 14, 15])
def test_gemm_tiled_direct_to_lds(variant):
    """The variants whose tiles go from global memory straight into LDS: K in whole steps of 64,
    fewer steps than stages, many steps (every stage is reused), ragged M and N."""
    for M, N, Kd in ((300, 530, 1024), (70, 260, 64), (513, 100, 192), (9, 700, 128), (257, 258, 2048)):
        # (the gated epilogue stores pairs of columns where the output's rows are an even number of
        # values long, N = 260, 100, 700, and single values otherwise; in either type)
        for epi, cdt in ((0, torch.float32), (2, torch.bfloat16), (1, torch.float32), (0, torch.bfloat16), (2, torch.float32)):
            run_gemm(K().gemm_tiled, M, N, Kd, epi, torch.bfloat16, torch.bfloat16, cdt, variant=variant)
    with pytest.raises(Exception, match="multiple"):
        run_gemm(K().gemm_tiled, 70, 64, 72, 0, torch.bfloat16, torch.bfloat16, torch.float32, variant=variant)


def test_gemm_refuses_what_it_cannot_do():
    k = K()
    a = torch.zeros(4, 12, dtype=torch.bfloat16, device=DEV)
    w = torch.zeros(8, 12, dtype=torch.bfloat16, device=DEV)
    c = torch.zeros(4, 8, device=DEV)
    with pytest.raises(k.KernelError):
        k.gemm_skinny(a, w, c)                       # K = 12 is no multiple of 8
    k.gemm(a, w, c)                                  # the dispatcher falls back to the float kernel
    with pytest.raises(k.KernelError):
        k.gemm_generic(a.cpu(), w, c)
    with pytest.raises(k.KernelError):
        k.gemm_generic(a, w, torch.zeros(4, 9, device=DEV))


# ------------------------------------------------------------------------------------------ attention
class PagedCase:
    """Sequences with dense float64 q/k/v, and the same k/v scattered over shuffled cache pages."""

    def __init__(self, H, G, d, lens_old, lens_new, dtype, seed=0, poison=True, scale_q=None):
        rng = np.random.default_rng(seed)
        self.H, self.G, self.d, self.dtype = H, G, d, dtype
        n = len(lens_old)
        self.totals = [a + b for a, b in zip(lens_old, lens_new)]
        self.lens_old, self.lens_new = lens_old, lens_new
        self.q = [rng.standard_normal((t, H, d)) for t in self.totals]
        self.k = [rng.standard_normal((t, G, d)) for t in self.totals]
        self.v = [rng.standard_normal((t, G, d)) for t in self.totals]
        if scale_q is not None:
            scale_q(self)
        max_pages = max((t + PAGE - 1) // PAGE for t in self.totals)
        n_pages = sum((t + PAGE - 1) // PAGE for t in self.totals) + 3
        perm = rng.permutation(n_pages)
        fill = float("nan") if poison else 0.0
        kp = torch.full((n_pages, G, PAGE, d), fill, dtype=torch.float32)
        vp = torch.full((n_pages, G, d, PAGE), fill, dtype=torch.float32)
        table = torch.zeros((n + 2, max_pages), dtype=torch.int32)
        self.slots = list(rng.permutation(n + 2)[:n])
        nxt = 0
        for i, t in enumerate(self.totals):
            for j in range((t + PAGE - 1) // PAGE):
                pg = int(perm[nxt]); nxt += 1
                table[self.slots[i], j] = pg
                m = min(PAGE, t - j * PAGE)
                kp[pg, :, :m, :] = torch.from_numpy(self.k[i][j * PAGE:j * PAGE + m]).permute(1, 0, 2).float()
                vp[pg, :, :, :m] = torch.from_numpy(self.v[i][j * PAGE:j * PAGE + m]).permute(1, 2, 0).float()
        # plain arrays above; the kernels keep some pages in an order of their own
        self.k_pages, self.v_pages = K().kv_pages_pack(kp.to(dtype).to(DEV), vp.to(dtype).to(DEV))
        self.table_host = table
        self.table = table.to(DEV)
        # what the kernel sees after rounding to its storage type
        rd = lambda x: torch.from_numpy(x).to(dtype).double().numpy()
        self.q = [rd(x) for x in self.q]
        self.k = [rd(x) for x in self.k]
        self.v = [rd(x) for x in self.v]
        qnew = np.concatenate([q[o:] for q, o in zip(self.q, lens_old)])
        self.q_dev = torch.from_numpy(qnew).reshape(-1, H * d).to(dtype).to(DEV)

    def batch(self):
        from plan_reference import StepBatch
        toks = [[0] * n for n in self.lens_new]
        return StepBatch([int(s) for s in self.slots], self.lens_old, toks, [[] for _ in toks], 10, DEV)

    def reference(self, window=0):
        outs = []
        for q, k, v, o in zip(self.q, self.k, self.v, self.lens_old):
            outs.append(P.causal_attention(q, k, v, window)[o:])
        return np.concatenate(outs).reshape(-1, self.H * self.d)


ATTN_SHAPES = [(4, 2, 16), (6, 6, 32), (3, 1, 32), (8, 2, 64), (32, 8, 128), (5, 5, 128), (2, 1, 256), (40, 1, 64),
               (6, 2, 96), (6, 3, 160), (8, 4, 192), (4, 1, 224), (3, 3, 48),
               (4, 2, 320), (2, 1, 264), (3, 1, 512), (2, 2, 1024)]     # wider than a piece of 256 columns


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d", ATTN_SHAPES)
@pytest.mark.parametrize("window", [0, 70])
def test_attention_prefill(dtype, H, G, d, window):
    case = PagedCase(H, G, d, [0, 0, 5, 130], [1, 200, 67, 33], dtype, seed=H + d)
    b = case.batch()
    out = torch.zeros_like(case.q_dev)
    K().attn_prefill(case.q_dev, case.k_pages, case.v_pages, out, b, case.table, case.table.shape[1], H, G, d,
                     window, 1.0 / math.sqrt(d))
    ref = case.reference(window)
    err = np.abs(out.double().cpu().numpy() - ref).max()
    assert err <= tol(dtype, np.abs(ref).max()), err


@pytest.mark.parametrize("H,G,d,old,new", [(64, 16, 32, [0, 100], [700, 400]), (32, 16, 64, [0, 37], [1500, 640])])
def test_attention_prefill_with_more_tiles_than_places(H, G, d, old, new):
    """Up to two workgroups a CU the matrix-core kernel runs eight waves, in two halves that share
    a tile's pages; with more tiles than that four waves.  The other prefill tests are small and
    take the first way, this one is large enough (more than 512 workgroups) for the second."""
    case = PagedCase(H, G, d, old, new, torch.bfloat16, seed=H + d)
    b = case.batch()
    heads = 4 if H // G >= 3 else H // G              # heads of a group that share a workgroup
    n_tiles = sum(-(-n // (32 * (4 // heads))) for n in new)
    assert n_tiles * G * -(-(H // G) // heads) > 512
    out = torch.zeros_like(case.q_dev)
    K().attn_prefill(case.q_dev, case.k_pages, case.v_pages, out, b, case.table, case.table.shape[1], H, G, d,
                     0, 1.0 / math.sqrt(d))
    ref = case.reference(0)
    err = np.abs(out.double().cpu().numpy() - ref).max()
    assert err <= tol(torch.bfloat16, np.abs(ref).max()), err


@pytest.mark.parametrize("H,G,d", [(6, 6, 32), (8, 2, 64), (32, 8, 128), (40, 1, 64), (6, 2, 96), (4, 2, 192), (2, 1, 256)])
@pytest.mark.parametrize("style", ["pairwise", "half", None])
@pytest.mark.parametrize("window", [0, 70])
def test_attention_prefill_with_rotation_inside(H, G, d, style, window):
    """The prefill step of the matrix-core path: the rotation kernel writes only keys and values
    (no rotated copy of q), and the attention kernel takes q unrotated in float and rotates it on
    the way in.  New tokens that start a sequence, continue one inside a page and across pages;
    their cache rows hold NaN beforehand."""
    old, new = [0, 0, 5, 130], [1, 200, 67, 33]
    case = PagedCase(H, G, d, old, new, torch.bfloat16, seed=H + d)
    b = case.batch()
    T = sum(new)
    rng = np.random.default_rng(11)
    qkv = rng.standard_normal((T, (H + 2 * G) * d)).astype(np.float32)
    inv = P.rope_inv_freq(d, 10000.0)
    positions = np.concatenate([np.arange(o, o + n) for o, n in zip(old, new)])
    cos, sin = P.rope_tables(np.arange(256), inv)
    x = qkv.astype(np.float64).reshape(T, H + 2 * G, d)
    if style is None:
        q_ref, k_ref = x[:, :H], x[:, H:H + G]
    else:
        c, s = P.rope_tables(positions, inv)
        q_ref, k_ref = P.apply_rope(x[:, :H], c, s, style), P.apply_rope(x[:, H:H + G], c, s, style)
    v_ref = x[:, H + G:]
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(torch.bfloat16)
    row = 0
    for i, (o, n) in enumerate(zip(old, new)):
        case.q[i][o:] = bf(q_ref[row:row + n]).double().numpy()
        case.k[i][o:] = bf(k_ref[row:row + n]).double().numpy()
        case.v[i][o:] = bf(v_ref[row:row + n]).double().numpy()
        row += n
    ref = case.reference(window)
    tok_page = b.write_pages(0, case.table_host, case.table_host.shape[1])
    k_plain, v_plain = K().kv_pages_unpack(case.k_pages, case.v_pages)
    for t in range(T):
        k_plain[int(tok_page[t]), :, positions[t] % PAGE, :] = float("nan")
        v_plain[int(tok_page[t]), :, :, positions[t] % PAGE] = float("nan")
    case.k_pages, case.v_pages = K().kv_pages_pack(k_plain, v_plain)
    dev = lambda t: None if style is None else torch.from_numpy(t).float().to(DEV)
    st = 0 if style != "half" else 1
    qkv_dev = torch.from_numpy(qkv).to(DEV)
    K().kv_store_tiles(qkv_dev, case.k_pages, case.v_pages, dev(cos), dev(sin), st, b, case.table, case.table.shape[1], H, G, d)
    out = torch.zeros(T, H * d, dtype=torch.bfloat16, device=DEV)
    K().attn_prefill_rope(qkv_dev, case.k_pages, case.v_pages, out, b, case.table, case.table.shape[1], H, G, d, window,
                          1.0 / math.sqrt(d), dev(cos), dev(sin), st)
    err = np.abs(out.double().cpu().numpy() - ref).max()
    assert err <= tol(torch.bfloat16, np.abs(ref).max()), err
    k_plain, v_plain = K().kv_pages_unpack(case.k_pages, case.v_pages)
    for t in range(T):
        pg, r = int(tok_page[t]), positions[t] % PAGE
        # (a key rotated in 32-bit and one rotated in 64-bit may round to neighbouring bfloat16 values)
        assert np.abs(k_plain[pg, :, r, :].double().cpu().numpy() - k_ref[t]).max() <= tol(torch.bfloat16, 4.0)
        assert torch.equal(v_plain[pg, :, :, r].cpu(), bf(v_ref[t]))


def decode_work_list(case, window, pages_per_chunk, spare=0):
    """The work list the engine would build, with room for `spare` more entries behind it (a
    recorded step's list has room for full-length sequences): those hold garbage."""
    from plan_reference import decode_chunk_list, with_header
    b = case.batch()
    entries, most = decode_chunk_list(b.slots, b.pos0, window, pages_per_chunk, case.table_host,
                                      case.table_host.shape[1])
    n_live = len(entries)
    if spare:
        entries = np.concatenate([entries, np.full((spare, 8), 12345, np.int32)])
    return torch.from_numpy(with_header(entries, n_live)).to(DEV), len(entries), most


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("H,G,d", ATTN_SHAPES)
@pytest.mark.parametrize("pages_per_chunk,window,spare", [(64, 0, 0), (4, 0, 3), (1, 0, 0), (2, 100, 1), (3, 200, 0)])
def test_attention_decode(dtype, H, G, d, pages_per_chunk, window, spare):
    pos0 = [0, 63, 64, 700, 129]
    case = PagedCase(H, G, d, pos0, [1, 1, 1, 1, 1], dtype, seed=H * d + pages_per_chunk)
    b = case.batch()
    out = torch.zeros_like(case.q_dev)
    chunk_list, n_chunks, most = decode_work_list(case, window, pages_per_chunk, spare)
    partial = torch.full((b.n_seq * H * most * (d + 2),), float("nan"), device=DEV)
    K().attn_decode(case.q_dev, case.k_pages, case.v_pages, out, partial, b.n_seq, chunk_list, n_chunks,
                    pages_per_chunk, most, b.seq_pos0, case.table, case.table.shape[1], H, G, d, window,
                    1.0 / math.sqrt(d))
    ref = case.reference(window)
    err = np.abs(out.double().cpu().numpy() - ref).max()
    assert err <= tol(dtype, np.abs(ref).max()), err
    # the same with the chunks combined by the attention kernel itself (kernels that cannot ignore
    # the counters); twice, for the counters must be left at zero
    done = torch.zeros(K().attn_decode_counters(b.n_seq, H, G), dtype=torch.int32, device=DEV)
    for _ in range(2):
        out.zero_()
        partial.fill_(float("nan"))
        K().attn_decode(case.q_dev, case.k_pages, case.v_pages, out, partial, b.n_seq, chunk_list, n_chunks,
                        pages_per_chunk, most, b.seq_pos0, case.table, case.table.shape[1], H, G, d, window,
                        1.0 / math.sqrt(d), done)
        err = np.abs(out.double().cpu().numpy() - ref).max()
        assert err <= tol(dtype, np.abs(ref).max()), err
        assert not done.any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("pages_per_chunk", [32, 64])
def test_attention_decode_over_long_chunks(dtype, pages_per_chunk):
    """Chunks of 32 and 64 pages, as long contexts get them: a wave walks over up to 16 tiles, most
    of whose pages it looks up in the page table itself (a work list's entry carries four), and a
    sequence of 64 pages is two chunks of 32 or one of 64; shorter sequences beside it."""
    H, G, d = 8, 2, 128
    pos0 = [4095, 2049, 70, 1984]
    case = PagedCase(H, G, d, pos0, [1] * len(pos0), dtype, seed=pages_per_chunk)
    b = case.batch()
    ref = case.reference(0)
    chunk_list, n_chunks, most = decode_work_list(case, 0, pages_per_chunk, spare=2)
    partial = torch.full((b.n_seq * H * most * (d + 2),), float("nan"), device=DEV)
    done = torch.zeros(K().attn_decode_counters(b.n_seq, H, G), dtype=torch.int32, device=DEV)
    for counters in (None, done):
        out = torch.zeros_like(case.q_dev)
        args = (case.q_dev, case.k_pages, case.v_pages, out, partial, b.n_seq, chunk_list, n_chunks, pages_per_chunk, most,
                b.seq_pos0, case.table, case.table.shape[1], H, G, d, 0, 1.0 / math.sqrt(d))
        K().attn_decode(*args) if counters is None else K().attn_decode(*args, counters)
        err = np.abs(out.double().cpu().numpy() - ref).max()
        assert err <= tol(dtype, np.abs(ref).max()), err
    assert not done.any()


@pytest.mark.parametrize("d", [64, 128])
@pytest.mark.parametrize("pages_per_chunk", [1, 4, 8])
def test_attention_decode_many_sequences(d, pages_per_chunk):
    """With many sequences the matrix-core kernel runs four waves a workgroup instead of eight."""
    H, G = 16, 8
    rng = np.random.default_rng(d + pages_per_chunk)
    pos0 = [int(x) for x in rng.integers(0, 900, size=40)]
    case = PagedCase(H, G, d, pos0, [1] * len(pos0), torch.bfloat16, seed=d)
    b = case.batch()
    out = torch.zeros_like(case.q_dev)
    chunk_list, n_chunks, most = decode_work_list(case, 0, pages_per_chunk, spare=2)
    partial = torch.full((b.n_seq * H * most * (d + 2),), float("nan"), device=DEV)
    done = torch.zeros(K().attn_decode_counters(b.n_seq, H, G), dtype=torch.int32, device=DEV)
    ref = case.reference(0)
    outs = []
    # the partial results hold NaN before every run: one that is read before it arrived shows
    for counters in [None] + [done] * 12:
        out.zero_()
        partial.fill_(float("nan"))
        K().attn_decode(case.q_dev, case.k_pages, case.v_pages, out, partial, b.n_seq, chunk_list, n_chunks,
                        pages_per_chunk, most, b.seq_pos0, case.table, case.table.shape[1], H, G, d, 0,
                        1.0 / math.sqrt(d), counters)
        err = np.abs(out.double().cpu().numpy() - ref).max()
        assert err <= tol(torch.bfloat16, np.abs(ref).max()), err
        assert not done.any()
        outs.append(out.clone())
    for o in outs[2:]:
        assert torch.equal(outs[1], o)            # whichever workgroup came last, the sum is the same


@pytest.mark.parametrize("H,G,d", [(6, 6, 32), (8, 2, 64), (32, 8, 128), (40, 1, 64), (6, 2, 96), (4, 2, 160), (2, 1, 256)])
@pytest.mark.parametrize("style", ["pairwise", "half", None])
@pytest.mark.parametrize("pages_per_chunk,window", [(4, 0), (1, 0), (16, 0), (2, 100), (4, 1)])
def test_attention_decode_with_rotation_and_cache_write_inside(H, G, d, style, pages_per_chunk, window):
    """The one-launch decode step: q, k, v of the new tokens come unrotated in float; the kernel
    must give what rotation + cache write + attention give, and leave the same rows in the cache.
    The cache rows of the new tokens hold NaN beforehand: they must not be read.  Positions at the
    start of a sequence, at a page's first and last row, and deep into a sequence."""
    pos0 = [0, 63, 64, 700, 129, 31, 32]
    n = len(pos0)
    case = PagedCase(H, G, d, pos0, [1] * n, torch.bfloat16, seed=H + d + pages_per_chunk)
    b = case.batch()
    rng = np.random.default_rng(7)
    qkv = rng.standard_normal((n, (H + 2 * G) * d)).astype(np.float32)
    inv = P.rope_inv_freq(d, 10000.0)
    cos, sin = P.rope_tables(np.arange(800), inv)
    x = qkv.astype(np.float64).reshape(n, H + 2 * G, d)
    if style is None:
        q_ref, k_ref = x[:, :H], x[:, H:H + G]
    else:
        c, s = P.rope_tables(np.asarray(pos0), inv)
        q_ref, k_ref = P.apply_rope(x[:, :H], c, s, style), P.apply_rope(x[:, H:H + G], c, s, style)
    v_ref = x[:, H + G:]
    bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(torch.bfloat16)
    # the reference: the paged case with its last key and value replaced by the new token's
    for i in range(n):
        case.q[i][-1] = bf(q_ref[i]).double().numpy()
        case.k[i][-1] = bf(k_ref[i]).double().numpy()
        case.v[i][-1] = bf(v_ref[i]).double().numpy()
    ref = case.reference(window)
    # poison the new tokens' cache rows
    tok_page = b.write_pages(0, case.table_host, case.table_host.shape[1])
    k_plain, v_plain = K().kv_pages_unpack(case.k_pages, case.v_pages)
    for i in range(n):
        pg, row = int(tok_page[i]), pos0[i] % PAGE
        k_plain[pg, :, row, :] = float("nan")
        v_plain[pg, :, :, row] = float("nan")
    case.k_pages, case.v_pages = K().kv_pages_pack(k_plain, v_plain)
    out = torch.zeros(n, H * d, dtype=torch.bfloat16, device=DEV)
    chunk_list, n_chunks, most = decode_work_list(case, window, pages_per_chunk, spare=1)
    partial = torch.full((n * H * most * (d + 2),), float("nan"), device=DEV)
    dev = lambda t: None if style is None else torch.from_numpy(t).float().to(DEV)
    # with a second kernel combining the chunks, then with the attention kernel doing it itself
    # (the second call finds the new tokens' rows written; it must give the same)
    done = torch.zeros(K().attn_decode_counters(n, H, G), dtype=torch.int32, device=DEV)
    for counters in (None, done):
        out.zero_()
        K().attn_decode_rope(torch.from_numpy(qkv).to(DEV), case.k_pages, case.v_pages, out, partial, n, chunk_list,
                             n_chunks, pages_per_chunk, most, b.seq_pos0, case.table, case.table.shape[1], H, G, d,
                             window, 1.0 / math.sqrt(d), dev(cos), dev(sin), 0 if style != "half" else 1, tok_page,
                             counters)
        err = np.abs(out.double().cpu().numpy() - ref).max()
        assert err <= tol(torch.bfloat16, np.abs(ref).max()), err
        assert not done.any()
    k_plain, v_plain = K().kv_pages_unpack(case.k_pages, case.v_pages)
    for i in range(n):
        pg, row = int(tok_page[i]), pos0[i] % PAGE
        if style is None:
            assert torch.equal(k_plain[pg, :, row, :].cpu(), bf(k_ref[i]))
        else:       # (a key rotated in 32-bit and one rotated in 64-bit may round to neighbouring bfloat16 values)
            assert np.abs(k_plain[pg, :, row, :].double().cpu().numpy() - k_ref[i]).max() <= tol(torch.bfloat16, 4.0)
        assert torch.equal(v_plain[pg, :, :, row].cpu(), bf(v_ref[i]))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_finds_a_far_key(dtype):
    """One key among hundreds is made to dominate: the output must be its value row.  A kernel
    that drops a page, a split or the window's edge returns something else."""
    H, G, d = 4, 2, 64
    target = 130

    def boost(c):
        for i in range(len(c.totals)):
            if c.totals[i] > target:
                c.k[i][target] = 0.0
                c.k[i][target, :, 0] = 30.0
                c.q[i][-1] = 0.0
                c.q[i][-1, :, 0] = 30.0
    case = PagedCase(H, G, d, [699], [1], dtype, seed=3, scale_q=boost)
    b = case.batch()
    for pages_per_chunk in (16, 4, 1):
        out = torch.zeros_like(case.q_dev)
        chunk_list, n_chunks, most = decode_work_list(case, 0, pages_per_chunk)
        partial = torch.zeros(b.n_seq * H * most * (d + 2), device=DEV)
        K().attn_decode(case.q_dev, case.k_pages, case.v_pages, out, partial, 1, chunk_list, n_chunks,
                        pages_per_chunk, most, b.seq_pos0, case.table, case.table.shape[1], H, G, d, 0,
                        1.0 / math.sqrt(d))
        got = out.double().cpu().numpy().reshape(H, d)
        for h in range(H):
            assert np.abs(got[h] - case.v[0][target, h // 2]).max() < 2e-2


@pytest.mark.parametrize("pages_per_chunk", [32, 64])
@pytest.mark.parametrize("where", ["fifth page of a chunk", "last page of a chunk", "second chunk"])
def test_attention_finds_a_far_key_in_a_long_chunk(pages_per_chunk, where):
    """Chunks of 32 and 64 pages: a work list's entry carries a chunk's first four pages and the
    matrix-core kernel looks the others up in the page table itself.  The key that dominates lies
    in such a page: the fifth of the first chunk, the chunk's last, or a page past the fourth of
    the second chunk, whose partial result is merged.  A wrong or dropped page gives another
    value row.  With a second kernel merging the chunks, with the attention kernel merging them
    itself, and in the kernel that also takes the new token unrotated and writes it to the cache."""
    H, G, d = 8, 2, 128
    n_old = 64 * (pages_per_chunk + 30) - 7              # two chunks of 64 pages, three of 32
    page = {"fifth page of a chunk": 4, "last page of a chunk": pages_per_chunk - 1, "second chunk": pages_per_chunk + 6}[where]
    target = 64 * page + 37

    def boost(c):
        c.k[0][target] = 0.0
        c.k[0][target, :, 0] = 30.0
        c.q[0][-1] = 0.0
        c.q[0][-1, :, 0] = 30.0
    case = PagedCase(H, G, d, [n_old], [1], torch.bfloat16, seed=pages_per_chunk, scale_q=boost)
    b = case.batch()
    chunk_list, n_chunks, most = decode_work_list(case, 0, pages_per_chunk, spare=1)
    assert most >= 2
    partial = torch.full((H * most * (d + 2),), float("nan"), device=DEV)
    done = torch.zeros(K().attn_decode_counters(1, H, G), dtype=torch.int32, device=DEV)

    def check(out):
        got = out.double().cpu().numpy().reshape(H, d)
        for h in range(H):
            assert np.abs(got[h] - case.v[0][target, h // (H // G)]).max() < 2e-2, (where, h)
    for counters in (None, done):
        out = torch.zeros_like(case.q_dev)
        K().attn_decode(case.q_dev, case.k_pages, case.v_pages, out, partial, 1, chunk_list, n_chunks, pages_per_chunk, most,
                        b.seq_pos0, case.table, case.table.shape[1], H, G, d, 0, 1.0 / math.sqrt(d), counters)
        check(out)
    # the one-launch kernel: q, k, v of the new token in float, no rotation
    qkv = torch.zeros(1, (H + 2 * G) * d, device=DEV)
    qkv[0, :H * d] = case.q_dev[0].float()
    qkv[0, H * d:(H + G) * d] = torch.from_numpy(case.k[0][-1].reshape(-1)).float().to(DEV)
    qkv[0, (H + G) * d:] = torch.from_numpy(case.v[0][-1].reshape(-1)).float().to(DEV)
    tok_page = b.write_pages(0, case.table_host, case.table_host.shape[1])
    for counters in (None, done):
        out = torch.zeros(1, H * d, dtype=torch.bfloat16, device=DEV)
        K().attn_decode_rope(qkv, case.k_pages, case.v_pages, out, partial, 1, chunk_list, n_chunks, pages_per_chunk, most,
                             b.seq_pos0, case.table, case.table.shape[1], H, G, d, 0, 1.0 / math.sqrt(d), None, None, 0,
                             tok_page, counters)
        check(out)
    assert not done.any()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_over_pages_beyond_four_gigabytes(dtype):
    """A cache of a large batch of long sequences: the pages of this case lie more than 2^32 bytes
    (and more than 2^31 elements) into the key and value arrays.  An offset computed in 32 bits
    anywhere (the table's page times the page's size) reads or writes somewhere else."""
    H, G, d = 32, 8, 128
    page_bytes = G * PAGE * d * (4 if dtype == torch.float32 else 2)
    base = (1 << 32) // page_bytes + 777
    case = PagedCase(H, G, d, [0, 130, 650], [70, 33, 1], dtype, seed=5)

    def moved(pages):
        big = torch.empty((base + pages.shape[0],) + tuple(pages.shape[1:]), dtype=dtype, device=DEV)
        big[:64].fill_(float("nan"))          # where a truncated offset of these pages would land
        big[base:] = pages
        return big
    k_big, v_big = moved(case.k_pages), moved(case.v_pages)
    table_host = case.table_host + base
    table = table_host.to(DEV)
    b = case.batch()
    ref = case.reference(0)
    out = torch.zeros_like(case.q_dev)
    K().attn_prefill(case.q_dev, k_big, v_big, out, b, table, table.shape[1], H, G, d, 0, 1.0 / math.sqrt(d))
    err = np.abs(out.double().cpu().numpy() - ref).max()
    assert err <= tol(dtype, np.abs(ref).max()), err
    # the last sequence alone as a decode step, its chunks combined by the kernel and by the merge kernel
    from plan_reference import StepBatch, decode_chunk_list, with_header
    slot, pos0 = int(case.slots[2]), 650
    db = StepBatch([slot], [pos0], [[0]], [[]], 10, DEV)
    q1 = case.q_dev[-1:].contiguous()
    for pages_per_chunk in (16, 2):
        entries, most = decode_chunk_list(db.slots, db.pos0, 0, pages_per_chunk, table_host, table_host.shape[1])
        chunk_list = torch.from_numpy(with_header(entries, len(entries))).to(DEV)
        partial = torch.full((H * most * (d + 2),), float("nan"), device=DEV)
        done = torch.zeros(K().attn_decode_counters(1, H, G), dtype=torch.int32, device=DEV)
        for counters in (None, done):
            out1 = torch.zeros_like(q1)
            args = (q1, k_big, v_big, out1, partial, 1, chunk_list, len(entries), pages_per_chunk, most, db.seq_pos0,
                    table, table.shape[1], H, G, d, 0, 1.0 / math.sqrt(d))
            K().attn_decode(*args) if counters is None else K().attn_decode(*args, counters)
            err = np.abs(out1.double().cpu().numpy() - ref[-1:]).max()
            assert err <= tol(dtype, np.abs(ref).max()), (pages_per_chunk, err)
    if dtype == torch.bfloat16:
        # the decode step's one launch: rotation, cache write and attention; the new token's row must land
        # in its page up there, and the output must be that of the sequence with this last token
        rng = np.random.default_rng(2)
        qkv1 = rng.standard_normal((1, (H + 2 * G) * d)).astype(np.float32)
        inv = P.rope_inv_freq(d, 10000.0)
        cos, sin = P.rope_tables(np.arange(800), inv)
        c, s_ = P.rope_tables(np.asarray([pos0]), inv)
        x = qkv1.astype(np.float64).reshape(1, H + 2 * G, d)
        bf = lambda t: torch.from_numpy(np.ascontiguousarray(t)).to(torch.bfloat16)
        q_new, k_new, v_new = P.apply_rope(x[:, :H], c, s_, "half")[0], P.apply_rope(x[:, H:H + G], c, s_, "half")[0], x[0, H + G:]
        case.q[2][-1], case.k[2][-1], case.v[2][-1] = (bf(t).double().numpy() for t in (q_new, k_new, v_new))
        ref1 = P.causal_attention(case.q[2], case.k[2], case.v[2], 0)[-1:].reshape(1, H * d)
        tok_page = db.write_pages(0, table_host, table_host.shape[1])
        assert int(tok_page[0]) >= base
        entries, most = decode_chunk_list(db.slots, db.pos0, 0, 4, table_host, table_host.shape[1])
        chunk_list = torch.from_numpy(with_header(entries, len(entries))).to(DEV)
        partial = torch.full((H * most * (d + 2),), float("nan"), device=DEV)
        out1 = torch.zeros(1, H * d, dtype=dtype, device=DEV)
        K().attn_decode_rope(torch.from_numpy(qkv1).to(DEV), k_big, v_big, out1, partial, 1, chunk_list, len(entries), 4,
                             most, db.seq_pos0, table, table.shape[1], H, G, d, 0, 1.0 / math.sqrt(d),
                             torch.from_numpy(cos).float().to(DEV), torch.from_numpy(sin).float().to(DEV), 1, tok_page, done)
        err = np.abs(out1.double().cpu().numpy() - ref1).max()
        assert err <= tol(dtype, np.abs(ref1).max()), err
        pg = int(tok_page[0])
        kp, vp = K().kv_pages_unpack(k_big[pg:pg + 1], v_big[pg:pg + 1])
        assert torch.equal(kp[0, :, pos0 % PAGE, :].cpu(), bf(k_new)) and torch.equal(vp[0, :, :, pos0 % PAGE].cpu(), bf(v_new))
    # writing keys and values there: both kernels, read back through the plain order
    rng = np.random.default_rng(1)
    T = sum(case.lens_new)
    qkv = torch.from_numpy(rng.standard_normal((T, (H + 2 * G) * d)).astype(np.float32)).to(DEV)
    inv = P.rope_inv_freq(d, 1000.0)
    cos, sin = (torch.from_numpy(x).float().to(DEV) for x in P.rope_tables(np.arange(800), inv))
    positions = np.concatenate([np.arange(p, p + n) for p, n in zip(case.lens_old, case.lens_new)])
    c, s_ = P.rope_tables(positions, inv)
    x = qkv.double().cpu().numpy().reshape(T, H + 2 * G, d)
    k_ref, v_ref = P.apply_rope(x[:, H:H + G], c, s_, "half"), x[:, H + G:]
    seq_of = np.repeat(np.arange(3), case.lens_new)
    tab = table_host.numpy()
    for which in ("rope_kv_store", "kv_store_tiles"):
        k_big[base:].zero_()
        v_big[base:].zero_()
        if which == "rope_kv_store":
            q_out = torch.zeros(T, H * d, dtype=dtype, device=DEV)
            K().rope_kv_store(qkv, q_out, k_big, v_big, cos, sin, 1, b.tok_pos,
                              b.write_pages(0, table_host, table_host.shape[1]), H, G, d)
        else:
            K().kv_store_tiles(qkv, k_big, v_big, cos, sin, 1, b, table, table.shape[1], H, G, d)
        kp, vp = K().kv_pages_unpack(k_big[base:], v_big[base:])
        kp, vp = kp.double().cpu().numpy(), vp.double().cpu().numpy()
        for t in range(T):
            pg = tab[case.slots[seq_of[t]], positions[t] // PAGE] - base
            assert np.abs(kp[pg, :, positions[t] % PAGE, :] - k_ref[t]).max() <= tol(dtype, 4.0), (which, t)
            assert np.abs(vp[pg, :, :, positions[t] % PAGE] - v_ref[t]).max() <= tol(dtype, 4.0), (which, t)
    del k_big, v_big
    torch.cuda.empty_cache()


# ------------------------------------------------------------------------------------------ rope
@pytest.mark.parametrize("d", [16, 32, 48, 64, 96, 128, 160, 192, 224, 256])
def test_kv_page_order_is_a_permutation(d):
    """Every element of a page has one place; 32-bit pages and head sizes outside the matrix-core
    kernels' are plain arrays; packing and unpacking undo each other."""
    for dtype in (torch.float32, torch.bfloat16):
        k_idx, v_idx = K().kv_page_order(dtype, d)
        assert sorted(k_idx.reshape(-1).tolist()) == list(range(PAGE * d))
        assert sorted(v_idx.reshape(-1).tolist()) == list(range(PAGE * d))
        plain = dtype == torch.float32 or d % 32 != 0
        assert (k_idx.reshape(-1).tolist() == list(range(PAGE * d))) == plain
        assert (v_idx.reshape(-1).tolist() == list(range(PAGE * d))) == plain
        k = torch.randn(3, 2, PAGE, d).to(dtype).to(DEV)
        v = torch.randn(3, 2, d, PAGE).to(dtype).to(DEV)
        kp, vp = K().kv_pages_pack(k, v)
        k2, v2 = K().kv_pages_unpack(kp, vp)
        assert torch.equal(k, k2) and torch.equal(v, v2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("style", ["pairwise", "half"])
def test_rope_kv_store(dtype, style):
    from plan_reference import StepBatch
    H, G, d = 3, 1, 32
    rng = np.random.default_rng(0)
    slots, pos0, n_new = [2, 0], [61, 0], [5, 70]
    T = sum(n_new)
    qkv = rng.standard_normal((T, (H + 2 * G) * d)).astype(np.float32)
    inv = P.rope_inv_freq(d, 1000.0)
    b = StepBatch(slots, pos0, [[0] * n for n in n_new], [[], []], 10, DEV)
    positions = np.concatenate([np.arange(p, p + n) for p, n in zip(pos0, n_new)])
    cos, sin = P.rope_tables(np.arange(200), inv)
    table_host = torch.tensor([[4, 1], [0, 0], [3, 5]], dtype=torch.int32)
    table = table_host.to(DEV)
    kp = torch.zeros(6, G, PAGE, d, dtype=dtype, device=DEV)
    vp = torch.zeros(6, G, d, PAGE, dtype=dtype, device=DEV)
    q_out = torch.zeros(T, H * d, dtype=dtype, device=DEV)
    K().rope_kv_store(torch.from_numpy(qkv).to(DEV), q_out, kp, vp, torch.from_numpy(cos).float().to(DEV),
                      torch.from_numpy(sin).float().to(DEV), 0 if style == "pairwise" else 1, b.tok_pos,
                      b.write_pages(0, table_host, 2), H, G, d)
    x = qkv.astype(np.float64).reshape(T, H + 2 * G, d)
    c, s = P.rope_tables(positions, inv)
    q_ref = P.apply_rope(x[:, :H], c, s, style).reshape(T, H * d)
    k_ref = P.apply_rope(x[:, H:H + G], c, s, style)
    v_ref = x[:, H + G:]
    t_ = tol(dtype, 4.0)
    assert np.abs(q_out.double().cpu().numpy() - q_ref).max() <= t_
    kp, vp = K().kv_pages_unpack(kp, vp)
    kp, vp, tab = kp.double().cpu().numpy(), vp.double().cpu().numpy(), table.cpu().numpy()
    seq_of = np.repeat(np.arange(2), n_new)
    for t in range(T):
        pg = tab[slots[seq_of[t]], positions[t] // PAGE]
        assert np.abs(kp[pg, :, positions[t] % PAGE, :] - k_ref[t]).max() <= t_
        assert np.abs(vp[pg, :, :, positions[t] % PAGE] - v_ref[t]).max() <= t_
    # the kernel that writes only keys and values, tile by tile (values in runs of eight keys where
    # the tokens fill one: the first sequence starts at 61, the second at 0)
    kp2 = torch.zeros(6, G, PAGE, d, dtype=dtype, device=DEV)
    vp2 = torch.zeros(6, G, d, PAGE, dtype=dtype, device=DEV)
    K().kv_store_tiles(torch.from_numpy(qkv).to(DEV), kp2, vp2, torch.from_numpy(cos).float().to(DEV),
                       torch.from_numpy(sin).float().to(DEV), 0 if style == "pairwise" else 1, b, table, 2, H, G, d)
    kp2, vp2 = K().kv_pages_unpack(kp2, vp2)
    assert np.abs(kp2.double().cpu().numpy() - kp).max() <= t_ and np.array_equal(vp2.double().cpu().numpy(), vp)


# ------------------------------------------------------------------------------------------ sampling
def test_argmax_first_maximum():
    lg = torch.zeros(3, 1001)
    lg[0, 17] = lg[0, 900] = 2.0
    lg[1, :] = -1.0
    lg[2, 1000] = 5.0
    out = torch.zeros(3, dtype=torch.int32, device=DEV)
    K().argmax(lg.to(DEV), out)
    assert out.tolist() == [17, 0, 1000]


@pytest.mark.parametrize("V,scale", [(131, 1.0), (5000, 0.5), (128256, 1.0)])
@pytest.mark.parametrize("opts", [(0.8, 0, 1.0, 0.0), (0.8, 40, 0.9, 0.05), (1.3, 0, 0.7, 0.0), (0.5, 7, 1.0, 0.2),
                                  (1.0, 0, 1.0, 0.3), (0.0, 0, 1.0, 0.0), (0.9, 1000, 0.95, 0.0), (1.0, 1, 1.0, 0.0),
                                  (0.7, 130, 1.0, 0.0), (1.1, 40, 1.0, 0.0)])
def test_sampler_equals_plain(V, scale, opts):
    from picolm_amd.sampling import Sampler, SamplingParams, stream_state
    T, k, p, mp = opts
    rng = np.random.default_rng(V)
    n = 5 if V > 10000 else 16
    logits = (rng.standard_normal((n, V)) * scale).astype(np.float32)
    logits[0, :] = 0.25                 # all equal
    logits[1, ::2] = logits[1, 1]       # many equal
    logits[2, 5] = 40.0                 # one dominates
    smp = Sampler(SamplingParams(T, k, p, mp, seed=7), n, DEV)
    lg = torch.from_numpy(logits).to(DEV)
    states = [stream_state(7, i) for i in range(n)]
    for _ in range(3):
        got = smp.sample(lg, list(range(n)))
        for i in range(n):
            want, states[i] = SP.sample(logits[i], T, k, p, mp, states[i])
            assert got[i] == want, (i, got[i], want)


@pytest.mark.parametrize("V", [131, 4096, 4097, 9000, 128256])
def test_sampler_sliced_and_one_workgroup_kernels_agree(V):
    """With a small top_k a row is cut into slices for many workgroups; one workgroup per row does
    the same work without scratch memory.  Both must draw the same tokens from the same states:
    rows with all logits equal, many equal, a dominant one, equal values across a slice's border."""
    k = K()
    rng = np.random.default_rng(V)
    n = 6
    logits = rng.standard_normal((n, V)).astype(np.float32)
    logits[0, :] = -1.5
    logits[1, ::3] = 2.0
    logits[2, V // 2] = 30.0
    logits[3, max(0, min(V, 4096) - 20):min(V, 4096 + 20)] = 3.25
    lg = torch.from_numpy(logits).to(DEV)
    for T, top_k, top_p, min_p in ((0.8, 40, 0.9, 0.05), (1.0, 5, 1.0, 0.0), (0.6, 64, 0.5, 0.0), (1.5, 100, 1.0, 0.01)):
        if top_k >= V:
            continue
        need = k.sample_scratch_bytes(n, V, T, top_k)
        assert need > 0
        scratch = torch.empty(need, dtype=torch.uint8, device=DEV)
        st_a = torch.arange(1, n + 1, dtype=torch.int64, device=DEV) * 2654435761
        st_b = st_a.clone()
        out_a = torch.zeros(n, dtype=torch.int32, device=DEV)
        out_b = torch.zeros(n, dtype=torch.int32, device=DEV)
        for _ in range(8):
            k.sample(lg, out_a, T, top_k, top_p, min_p, st_a, None, scratch)
            k.sample(lg, out_b, T, top_k, top_p, min_p, st_b, None, None)
            assert out_a.tolist() == out_b.tolist(), (V, T, top_k, top_p, min_p)
            assert torch.equal(st_a, st_b)
    assert k.sample_scratch_bytes(n, V, 0.0, 40) == 0 and k.sample_scratch_bytes(n, V, 0.8, 0) == 0


def test_sampler_streams_do_not_depend_on_the_batch():
    from picolm_amd.sampling import Sampler, SamplingParams
    rng = np.random.default_rng(0)
    logits = torch.from_numpy(rng.standard_normal((4, 300)).astype(np.float32)).to(DEV)
    a = Sampler(SamplingParams(1.0, seed=3), 4, DEV)
    b = Sampler(SamplingParams(1.0, seed=3), 4, DEV)
    full = [a.sample(logits, [0, 1, 2, 3]) for _ in range(4)]
    part = [b.sample(logits[[1, 3]], [1, 3]) for _ in range(4)]
    assert [[f[1], f[3]] for f in full] == part
