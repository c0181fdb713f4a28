"""Each HIP kernel alone against a plain float32 reference of the same operation, at sizes
other than the tiny models': head sizes in steps of 16, head counts and groups that are
no power of two, widths and vocabularies that are no power of two."""
import math

import pytest
import torch

import plain_qwen3 as plain

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]


def _tol(dtype, n_round=1):
    # float32: a few ulp over a reduction; bfloat16: half an ulp (2^-9) per rounding
    return 2e-5 if dtype == torch.float32 else 2.0 ** -8 * n_round


def _grouped(vc):
    """A V pool [pages, nkv, page, d] as the bfloat16 path keeps it: [pages, nkv, page / 8, d, 8], eight keys that
    follow each other side by side for every dim."""
    pages, nkv, page, d = vc.shape
    return vc.reshape(pages, nkv, page // 8, 8, d).transpose(3, 4).contiguous()


def _ungrouped(vg):
    pages, nkv, groups, d, _ = vg.shape
    return vg.transpose(3, 4).reshape(pages, nkv, groups * 8, d)


def _rand(shape, dtype, gen, scale=1.0):
    return (torch.randn(shape, generator=gen) * scale).to(dtype)


def test_lanes_exchange_across_powers_of_two():
    """The exchange between lanes that the reductions are built from (lane swaps and data-parallel
    moves instead of a trip through LDS): lane l gets lane l ^ 1, 2, 4, 8, 16, 32's value; the
    wave's sum is the sum in the order of the butterfly from 32 down to 1, the same bits in every lane."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(3)
    v = torch.randn(64, generator=g) * torch.logspace(-3, 3, 64)
    out = kernels.lane_xor_probe(v.to(DEV)).cpu()
    lanes = torch.arange(64)
    for i in range(6):
        assert torch.equal(out[i], v[lanes ^ (1 << i)]), i
    s = v.clone()
    for off in (32, 16, 8, 4, 2, 1):
        s = s + s[lanes ^ off]
    assert torch.equal(out[6], s) and len(set(out[6].tolist())) == 1
    assert torch.equal(out[7], torch.full((64,), float(v.max())))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("V,H,T", [(301, 72, 37), (1000, 4096, 5)])
def test_embed(dtype, V, H, T):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(1)
    table = _rand((V, H), dtype, g)
    ids = torch.randint(0, V, (T,), generator=g, dtype=torch.int32)
    ids[0], ids[-1] = 0, V - 1
    out = kernels.embed(table.to(DEV), ids.to(DEV)).cpu()
    assert torch.equal(out, table.float()[ids.long()])


@pytest.mark.parametrize("out_dtype", DTYPES)
@pytest.mark.parametrize("y_dtype", [None, torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,eps", [(9, 200, 1e-5), (3, 4096, 1e-6), (70, 33, 1e-3)])
def test_add_rmsnorm(out_dtype, y_dtype, T, H, eps):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(2)
    resid = _rand((T, H), torch.float32, g, 3.0)
    y = _rand((T, H), y_dtype, g, 2.0) if y_dtype is not None else None
    w = 1 + 0.2 * torch.randn(H, generator=g)
    s = resid + (y.float() if y is not None else 0)
    ref = plain.rms_norm(s.double(), w.double(), eps)
    r_dev = resid.to(DEV)
    out = kernels.add_rmsnorm(r_dev, y.to(DEV) if y is not None else None, w.to(DEV), eps, out_dtype)
    assert out.dtype == out_dtype
    err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(out_dtype), err
    # the sum is written back into the residual stream, exactly
    assert torch.equal(r_dev.cpu(), s)
    # with rows: only those rows, and the residual stream is left alone
    rows = torch.tensor([T - 1, 0, T // 2], dtype=torch.int32)
    r_dev = resid.to(DEV)
    out2 = kernels.add_rmsnorm(r_dev, y.to(DEV) if y is not None else None, w.to(DEV), eps, out_dtype,
                               rows=rows.to(DEV))
    assert torch.equal(r_dev.cpu(), resid)
    assert torch.equal(out2.cpu(), out.cpu()[rows.long()])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,I", [(13, 48), (5, 1001), (2, 12288)])
def test_silu_mul(dtype, T, I):
    """(13, 48) is the shape of the reference's own probe
    (/root/reference/tests/probes/attention_misc_precision_probe.rs)."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(4)
    gu = _rand((T, 2 * I), dtype, g, 2.0)
    ref = plain.swiglu(gu[:, :I].double(), gu[:, I:].double())
    lib = torch.nn.functional.silu(gu[:, :I].double()) * gu[:, I:].double()
    assert torch.allclose(ref, lib, rtol=1e-12, atol=1e-12)
    out = kernels.silu_mul(gu.to(DEV)).cpu().double()
    err = (out - ref).abs().max() / ref.abs().max()
    assert err < _tol(dtype), err


@pytest.mark.parametrize("in_dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16),
                                                (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K", [(1, 77, 130), (5, 509, 96), (67, 130, 33), (130, 64, 4096)])
def test_gemm_fixed_order(in_dtype, out_dtype, M, N, K):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(5)
    x = _rand((M, K), in_dtype, g)
    w = _rand((N, K), in_dtype, g, 0.1)
    ref = x.double() @ w.double().T
    y = kernels.gemm_tn(x.to(DEV), w.to(DEV), out_dtype=out_dtype)
    err = (y.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < (1e-5 if out_dtype == torch.float32 else 2.0 ** -8), err
    # a row's result does not depend on the rows beside it: bit-equal alone and in the batch
    y1 = kernels.gemm_tn(x[M // 2:M // 2 + 1].contiguous().to(DEV), w.to(DEV), out_dtype=out_dtype)
    assert torch.equal(y1.cpu()[0], y.cpu()[M // 2])
    if out_dtype == torch.float32:
        acc = torch.ones((M, N), dtype=torch.float32, device=DEV)
        kernels.gemm_tn(x.to(DEV), w.to(DEV), out=acc, accumulate=True)
        assert torch.allclose(acc.cpu(), y.cpu() + 1.0, rtol=0, atol=1e-5 * float(ref.abs().max()) + 1e-6)


@pytest.mark.parametrize("M", [1, 3, 8, 64, 200])
@pytest.mark.parametrize("N,K", [(509, 96), (1536, 4096), (4096, 1408)])
def test_linear_bf16(M, N, K):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(6)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, 0.05)
    ref = x.double() @ w.double().T
    y = kernels.linear_bf16(x.to(DEV), w.to(DEV))
    err = (y.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < 2.0 ** -8, err


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("M", [1, 5, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(509, 96), (77, 136), (1536, 4096), (4096, 1408), (16, 8)])
def test_linear_skinny(M, N, K, out_dtype):
    """The streaming matrix-core product for few rows: widths that are no multiple of the 16-row
    tile or the 32-wide k step, and every tile shape.  The order of the float32 sums is fixed by
    the number of waves alone: with the same waves, any number of row tiles and a row alone
    give bit-equal results."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(7)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, 0.05)
    ref = x.double() @ w.double().T
    tol = 2.0 ** -8 if out_dtype == torch.bfloat16 else 1e-5
    xd, wd = x.to(DEV), w.to(DEV)
    outs = {}
    shapes = [(0, 0), (1, 8), (2, 8), (3, 8), (4, 8), (6, 8), (1, 16), (2, 16)] + ([(8, 8)] if M <= 32 else [])
    for rt, nw in shapes:
        y = kernels.linear_skinny(xd, wd, out_dtype, row_tiles=rt, waves=nw)
        assert y.dtype == out_dtype and y.shape == (M, N)
        err = (y.cpu().double() - ref).abs().max() / ref.abs().max()
        assert err < tol, (rt, nw, err)
        outs[(rt, nw)] = y.cpu()
    for rt, nw in shapes:
        if nw == 8:
            assert torch.equal(outs[(1, 8)], outs[(rt, 8)]), rt
    assert torch.equal(outs[(1, 16)], outs[(2, 16)])
    r = M // 2
    for nw in (8, 16):
        y1 = kernels.linear_skinny(x[r:r + 1].contiguous().to(DEV), wd, out_dtype, waves=nw)
        assert torch.equal(y1.cpu()[0], outs[(1, nw)][r])
    # the default choice of waves comes from (N, K) alone: a row alone equals the row in the batch
    y0 = kernels.linear_skinny(x[r:r + 1].contiguous().to(DEV), wd, out_dtype)
    assert torch.equal(y0.cpu()[0], outs[(0, 0)][r])


@pytest.mark.parametrize("M", [1, 8, 40])
@pytest.mark.parametrize("N,K", [(4096, 4096), (320, 2048), (1000, 1544), (4096, 12288)])
def test_linear_skinny_partial_sums(M, N, K):
    """Narrow outputs may come back as float32 partial sums over slices of K; their sum is the
    product, the fused add + RMSNorm adds them in order, and a row's parts do not depend on the
    rows beside it."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(9)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, 0.05)
    ref = x.double() @ w.double().T
    parts = kernels.linear_skinny(x.to(DEV), w.to(DEV), allow_split=True)
    assert parts.dtype == torch.float32 and parts.dim() == 3 and parts.shape[1:] == (M, N) and parts.shape[0] > 1
    err = (parts.cpu().double().sum(0) - ref).abs().max() / ref.abs().max()
    assert err < 1e-5, err
    one = kernels.linear_skinny(x[M // 2:M // 2 + 1].contiguous().to(DEV), w.to(DEV), allow_split=True)
    assert torch.equal(one.cpu()[:, 0], parts.cpu()[:, M // 2])
    resid = _rand((M, N), torch.float32, g, 2.0)
    wn = 1 + 0.1 * torch.randn(N, generator=g)
    r_dev = resid.to(DEV)
    out = kernels.add_rmsnorm(r_dev, parts, wn.to(DEV), 1e-6, torch.bfloat16)
    s = resid.double() + ref
    want = plain.rms_norm(s, wn.double(), 1e-6)
    assert (out.cpu().double() - want).abs().max() / want.abs().max() < 2.0 ** -8
    assert (r_dev.cpu().double() - s).abs().max() / s.abs().max() < 1e-5


@pytest.mark.parametrize("M", [1, 8, 20, 64])
@pytest.mark.parametrize("I,K", [(224, 96), (176, 80), (1001, 136), (12288, 4096)])
def test_linear_skinny_gated(M, I, K):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(8)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((2 * I, K), torch.bfloat16, g, 0.1)
    gu = x.double() @ w.double().T
    ref = plain.swiglu(gu[:, :I], gu[:, I:])
    outs = []
    for rt in (0, 2, 4, 6) + ((8,) if M <= 32 else ()):
        y = kernels.linear_skinny(x.to(DEV), w.to(DEV), gated=True, row_tiles=rt, waves=8 if rt else 0)
        assert y.shape == (M, I)
        err = (y.cpu().double() - ref).abs().max() / ref.abs().max()
        assert err < 2.0 ** -8, (rt, err)
        outs.append(y.cpu())
    for y in outs[2:]:
        assert torch.equal(y, outs[1])     # the row tiles of a workgroup do not change a sum


@pytest.mark.parametrize("M", [1, 5, 16])
@pytest.mark.parametrize("N,K,N2", [(4096, 4096, 12288), (320, 136, 176), (1000, 1408, 509), (102 * 8, 96, 77)])
def test_linear_folded_norm(M, N, K, N2):
    """A norm between two products folded into them: the first adds into the float32 stream and
    hands on round(stream * g) with the rows' sums of squares in parts, the second scales its rows.
    Against add + RMSNorm + product in float64; the stream itself to float32 rounding."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(13)
    x = _rand((M, K), torch.bfloat16, g)
    w1 = _rand((N, K), torch.bfloat16, g, 0.05)
    resid = _rand((M, N), torch.float32, g, 2.0)
    gn = 1 + 0.2 * torch.randn(N, generator=g)
    eps = 1e-6
    r_dev = resid.to(DEV).clone()
    xg, ss = kernels.linear_fold_out(x.to(DEV), w1.to(DEV), r_dev, gn.to(DEV))
    want_r = resid.double() + x.double() @ w1.double().T
    assert (r_dev.cpu().double() - want_r).abs().max() / want_r.abs().max() < 1e-5
    assert ((ss.cpu().double().sum(1) - (want_r ** 2).sum(1)).abs() / (want_r ** 2).sum(1)).max() < 1e-5
    normed = plain.rms_norm(want_r, gn.double(), eps)
    for gated in (False, True):
        w2 = _rand(((2 if gated else 1) * N2, N), torch.bfloat16, g, 0.05)
        y = kernels.linear_fold_in(xg, ss, eps, w2.to(DEV), gated=gated)
        full = normed @ w2.double().T
        ref = plain.swiglu(full[:, :N2], full[:, N2:]) if gated else full
        err = (y.cpu().double() - ref).abs().max() / ref.abs().max()
        assert y.shape == (M, N2) and err < 2.0 ** -6, (gated, err)
    y32 = kernels.linear_fold_in(xg, ss, eps, w2[:N2].contiguous().to(DEV), out_dtype=torch.float32)
    ref = normed @ w2[:N2].double().T
    assert y32.dtype == torch.float32 and (y32.cpu().double() - ref).abs().max() / ref.abs().max() < 2.0 ** -6


@pytest.mark.parametrize("M", [1, 3, 4, 5, 8, 9, 16])
@pytest.mark.parametrize("N,K,N2", [(64, 256, 96), (300, 512, 70), (4096, 1024, 130), (1000, 2304, 64)])
def test_linear_thin_and_its_folded_norm(M, N, K, N2):
    """The thin product (few features a workgroup, whole sums, whole lines through LDS) in its
    three forms: plain, adding into the stream before a norm, scaling its rows after one; widths
    that are no multiple of the features a workgroup owns, one tile of K and an odd number of
    them, a row alone."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(19)
    x = _rand((M, K), torch.bfloat16, g)
    w1 = _rand((N, K), torch.bfloat16, g, 0.05)
    ref = x.double() @ w1.double().T
    for dt, tol in ((torch.bfloat16, 2.0 ** -8), (torch.float32, 1e-5)):
        y = kernels.linear_thin(x.to(DEV), w1.to(DEV), dt)
        assert y.dtype == dt and (y.cpu().double() - ref).abs().max() / ref.abs().max() < tol
        r = M // 2
        assert torch.equal(kernels.linear_thin(x[r:r + 1].contiguous().to(DEV), w1.to(DEV), dt)[0], y[r])
    resid = _rand((M, N), torch.float32, g, 2.0)
    gn = 1 + 0.2 * torch.randn(N, generator=g)
    eps = 1e-6
    r_dev = resid.to(DEV).clone()
    xg, ss = kernels.linear_thin_fold_out(x.to(DEV), w1.to(DEV), r_dev, gn.to(DEV))
    assert tuple(ss.shape) == (M, kernels.linear_thin_parts(N, K))
    want_r = resid.double() + ref
    assert (r_dev.cpu().double() - want_r).abs().max() / want_r.abs().max() < 1e-5
    assert ((ss.cpu().double().sum(1) - (want_r ** 2).sum(1)).abs() / (want_r ** 2).sum(1)).max() < 1e-5
    assert (xg.cpu().double() - want_r * gn.double()).abs().max() / (want_r * gn.double()).abs().max() < 2.0 ** -8
    if N % 256 == 0:
        normed = plain.rms_norm(want_r, gn.double(), eps)
        w2 = _rand((N2, N), torch.bfloat16, g, 0.05)
        y2 = kernels.linear_thin_fold_in(xg, ss, eps, w2.to(DEV))
        ref2 = normed @ w2.double().T
        assert y2.shape == (M, N2) and (y2.cpu().double() - ref2).abs().max() / ref2.abs().max() < 2.0 ** -6
        # the folded product of the streaming kernel takes the same operands
        y3 = kernels.linear_fold_in(xg, ss, eps, w2.to(DEV))
        assert (y3.cpu().double() - ref2).abs().max() / ref2.abs().max() < 2.0 ** -6


def test_linear_thin_refuses():
    from xinfer_amd import kernels
    x = torch.zeros((17, 256), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((32, 256), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(kernels.KernelError, match="1..16"):
        kernels.linear_thin(x, w)
    with pytest.raises(kernels.KernelError, match="multiple of 256"):
        kernels.linear_thin(x[:4, :128].contiguous(), w[:, :128].contiguous())
    assert kernels.linear_thin_parts(4096, 4096) == 256 and kernels.linear_thin_parts(5120, 5120) == 256
    assert kernels.linear_thin_parts(10240, 5120) == 512 and kernels.linear_thin_parts(64, 100) == 0


def test_linear_chooses_the_kernel_of_a_folded_product():
    """A product before a norm adds into the stream itself for up to 16 rows: with the thin kernel
    where K is a multiple of 256, else with the streaming kernel; more rows come back as partial
    sums of the tiled kernel for the norm to add."""
    from xinfer_amd import kernels
    from xinfer_amd.config.spec import PartSpec
    from xinfer_amd.parts.base import Folded, NormSink, norm_class
    from xinfer_amd.parts.linear import Linear
    g = torch.Generator().manual_seed(3)
    for N, K in ((256, 8192), (4096, 2048), (512, 1088)):
        lin = Linear(_rand((N, K), torch.bfloat16, g, 0.02).to(DEV))
        norm = norm_class("rmsnorm")(PartSpec("rmsnorm", dict(dim=N, eps=1e-6)), torch.bfloat16)
        norm.weight = torch.ones(N, device=DEV)
        for M in (4, 16, 40):
            x = _rand((M, K), torch.bfloat16, g).to(DEV)
            resid = torch.zeros((M, N), device=DEV)
            y = lin(x, allow_split=True, sink=NormSink(resid, norm))
            ref = x.cpu().double() @ lin.weight.cpu().double().T
            if M <= kernels.FOLD_ROWS:
                assert isinstance(y, Folded)
                thin = kernels.thin_ahead(M, lin.weight)
                assert thin == (K % 256 == 0)
                assert y.ss.shape[1] == (kernels.linear_thin_parts(N, K) if thin else kernels.linear_fold_parts(M, N, K))
                assert (resid.cpu().double() - ref).abs().max() / ref.abs().max() < 1e-5
            else:
                assert y.dtype == torch.float32 and tuple(y.shape) == (kernels.linear_mid_slices(N, K), M, N)
                assert float(resid.abs().max()) == 0.0
                assert (y.cpu().double().sum(0) - ref).abs().max() / ref.abs().max() < 1e-5


def test_linear_folded_norm_refuses():
    from xinfer_amd import kernels
    x = torch.zeros((17, 64), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((32, 64), dtype=torch.bfloat16, device=DEV)
    r = torch.zeros((17, 32), dtype=torch.float32, device=DEV)
    gw = torch.ones(32, device=DEV)
    with pytest.raises(kernels.KernelError, match="1..16"):
        kernels.linear_fold_out(x, w, r, gw)
    with pytest.raises(kernels.KernelError, match="do not match"):
        kernels.linear_fold_out(x[:4].contiguous(), w, r[:3].contiguous(), gw)
    with pytest.raises(kernels.KernelError, match="512 parts"):
        kernels.linear_fold_in(x[:4].contiguous(), torch.zeros((4, 600), device=DEV), 1e-6, w)


@pytest.mark.parametrize("M", [1, 17, 64, 65, 100, 128, 129, 200, 256])
@pytest.mark.parametrize("N,K", [(128, 64), (200, 256), (130, 1472), (4096, 1408), (640, 4096), (5120, 192)])
def test_linear_mid(M, N, K):
    """The tiled product for decode batches of up to 256 rows (blocks of 128) and narrow outputs:
    float32 partial sums in slices of K.  Widths that are no multiple of the 128-feature tile or of 4, a last
    tile of one feature's rows, slices of unequal length (K / 64 tiles dealt over the slices), a
    slice shorter than the depth of the copy pipeline; a row's values do not depend on the rows
    beside it, and rows past M leave nothing behind."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(11)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, 0.05)
    ref = x.double() @ w.double().T
    xd, wd = x.to(DEV), w.to(DEV)
    slices = kernels.linear_mid_slices(N, K)
    assert 1 <= slices <= K // 64
    y = kernels.linear_mid(xd, wd)
    assert y.dtype == torch.float32 and tuple(y.shape) == (slices, M, N)
    got = y.cpu().double().sum(0)
    err = (got - ref).abs().max() / ref.abs().max()
    assert err < 1e-5, err
    # each slice is the product over its own part of K: tiles of 64 dealt out as evenly as they go
    kt, lo = K // 64, 0
    for sl in range(slices):
        n = kt // slices + (1 if sl < kt % slices else 0)
        part = x[:, 64 * lo:64 * (lo + n)].double() @ w[:, 64 * lo:64 * (lo + n)].double().T
        assert (y[sl].cpu().double() - part).abs().max() / ref.abs().max() < 1e-5, sl
        lo += n
    assert lo == kt
    # the depth of the copy pipeline changes no bit
    for depth in (3, 4):
        assert torch.equal(kernels.linear_mid(xd, wd, depth=depth), y), depth
    # a row alone, and the first rows alone: the same bits
    r = M // 2
    y1 = kernels.linear_mid(xd[r:r + 1].contiguous(), wd)
    assert torch.equal(y1[:, 0], y[:, r])
    if M > 70:
        y70 = kernels.linear_mid(xd[:70].contiguous(), wd)
        assert torch.equal(y70, y[:, :70])


def test_linear_mid_refuses_and_serves_the_norm():
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(12)
    x = _rand((257, 128), torch.bfloat16, g).to(DEV)
    w = _rand((256, 128), torch.bfloat16, g).to(DEV)
    with pytest.raises(kernels.KernelError, match="1..256"):
        kernels.linear_mid(x, w)
    assert kernels.linear_mid_slices(256, 96) == 0 and kernels.linear_mid_slices(256, 32) == 0
    with pytest.raises(kernels.KernelError, match="multiple of 64"):
        kernels.linear_mid(x[:100, :96].contiguous(), w[:, :96].contiguous())
    # where a caller takes partial sums, rows 65..128 of a narrow product come from this kernel
    x, w = _rand((100, 1024), torch.bfloat16, g).to(DEV), _rand((640, 1024), torch.bfloat16, g, 0.05).to(DEV)
    y = kernels.linear_bf16(x, w, allow_split=True)
    assert y.dtype == torch.float32 and tuple(y.shape) == (kernels.linear_mid_slices(640, 1024), 100, 640)
    assert torch.equal(y, kernels.linear_mid(x, w))
    assert kernels.linear_bf16(x, w).shape == (100, 640)
    # the slices are chosen from (N, K) alone
    assert kernels.linear_mid_slices(4096, 12288) == 8 and kernels.linear_mid_slices(5120, 17408) == 6
    assert kernels.linear_mid_slices(151936, 4096) == 1
    # a wide output in float32 (the head) comes from the tiled kernel from 4 rows on, whole
    x, w = _rand((9, 128), torch.bfloat16, g).to(DEV), _rand((40000, 128), torch.bfloat16, g, 0.05).to(DEV)
    assert kernels.linear_mid_slices(40000, 128) == 1
    y = kernels.linear_bf16(x, w, torch.float32)
    assert y.dtype == torch.float32 and tuple(y.shape) == (9, 40000) and torch.equal(y, kernels.linear_mid(x, w)[0])
    ref = x.cpu().double() @ w.cpu().double().T
    assert (y.cpu().double() - ref).abs().max() / ref.abs().max() < 1e-5
    assert torch.equal(kernels.linear_bf16(x[:3].contiguous(), w, torch.float32), kernels.linear_skinny(x[:3].contiguous(), w, torch.float32))


@pytest.mark.parametrize("M", [1, 8, 16, 17, 32, 33, 64, 65, 128])
@pytest.mark.parametrize("N,K", [(64, 64), (100, 192), (182, 1024), (4100, 512), (1000, 4096)])
def test_linear_mid_gated(M, N, K):
    """The gated form of the tiled product: silu(x gate^T) * (x up^T), one rounding, for every
    shape of the kernel (up to 16, 32, 64 and 128 rows), widths that are no multiple of the
    features a workgroup owns, a last workgroup with a single feature; and the folded norm."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(13)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((2 * N, K), torch.bfloat16, g, 0.05)
    gate, up = x.double() @ w[:N].double().T, x.double() @ w[N:].double().T
    ref = gate / (1 + torch.exp(-gate)) * up
    y = kernels.linear_mid_gated(x.to(DEV), w.to(DEV))
    assert y.dtype == torch.bfloat16 and tuple(y.shape) == (M, N)
    assert (y.cpu().double() - ref).abs().max() / ref.abs().max() < 2.0 ** -8
    r = M // 2     # a row alone: the same bits
    assert torch.equal(kernels.linear_mid_gated(x[r:r + 1].contiguous().to(DEV), w.to(DEV))[0], y[r])
    if M <= 16:
        parts = 37
        ss = torch.rand((M, parts), generator=g) * 3 + 0.1
        eps = 1e-5
        inv = torch.rsqrt(ss.double().sum(1) / K + eps)[:, None]
        gs, us = gate * inv, up * inv
        want = gs / (1 + torch.exp(-gs)) * us
        yf = kernels.linear_mid_gated(x.to(DEV), w.to(DEV), ss.to(DEV), eps)
        assert (yf.cpu().double() - want).abs().max() / want.abs().max() < 2.0 ** -8
    else:
        with pytest.raises(kernels.KernelError, match="folded norm"):
            kernels.linear_mid_gated(x.to(DEV), w.to(DEV), torch.ones((M, 4), device=DEV), 1e-5)


@pytest.mark.parametrize("M", [1, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K,features", [(17408, 256, None), (25600, 128, None), (300, 320, 100), (129, 64, 128), (4100, 512, 65)])
def test_linear_mid_gated_wide_tile(M, N, K, features):
    """The gated product with up to 128 features a workgroup (a tile of 256 rows of w): chosen by
    itself from 17 to 64 rows where 64 features would make two rounds of workgroups (intermediate
    sizes of 17,408 and 25,600: 68 and 100 features), and forced here at other widths: a last
    workgroup of few features, waves without any, a single workgroup."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(14)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((2 * N, K), torch.bfloat16, g, 0.05)
    gate, up = x.double() @ w[:N].double().T, x.double() @ w[N:].double().T
    ref = gate / (1 + torch.exp(-gate)) * up
    if features is None:
        chosen = int(kernels.lib().xi_linear_mid_gated_features(N, M))
        assert chosen == ({17408: 68, 25600: 100}[N] if M > 16 else {17408: 34, 25600: 50}[N])
    y = kernels.linear_mid_gated(x.to(DEV), w.to(DEV), features=features)
    assert (y.cpu().double() - ref).abs().max() / ref.abs().max() < 2.0 ** -8
    narrow = kernels.linear_mid_gated(x.to(DEV), w.to(DEV), features=32)
    assert (y.float() - narrow.float()).abs().max() <= 2.0 ** -7 * ref.abs().max()      # the sums' order differs, no more
    if features is not None:
        with pytest.raises(kernels.KernelError, match="up to 64 rows"):
            kernels.linear_mid_gated(_rand((65, K), torch.bfloat16, g).to(DEV), w.to(DEV), features=features)


@pytest.mark.parametrize("M,N,K,slices", [(129, 4096, 4096, 8), (256, 4096, 12288, 8), (200, 1024, 3072, 1), (512, 4096, 12288, 8), (1000, 5120, 17408, 3), (256, 7168, 5120, 4), (300, 4096, 4096, 1), (128, 4096, 12288, 1), (256, 4096, 1024, 1), (1025, 4096, 12288, 1), (200, 1000, 2056, 1), (130, 6144, 2560, 5), (512, 2560, 9728, 6), (1024, 5120, 25600, 3), (256, 5120, 8192, 6), (256, 10240, 5120, 3)])
def test_tile_split_plan_and_the_sum_of_its_slices(M, N, K, slices):
    """Narrow products of 129 to 1,024 rows go to the many-row tiled kernel with K cut into slices:
    the chosen number of slices, the dispatch (`linear_bf16` with `allow_split`), every slice
    against a float64 product of its part of K, and the sum of the partial sums as the norm adds
    them."""
    from xinfer_amd import kernels
    assert kernels.tile_split_plan(M, N, K)[0] == slices
    g = torch.Generator().manual_seed(41)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, scale=0.05)
    ref = x.double() @ w.double().T
    y = kernels.linear_bf16(x.to(DEV), w.to(DEV), torch.bfloat16, allow_split=True)
    if slices > 1:
        assert y.shape == (slices, M, N) and y.dtype == torch.float32
        for sl in range(slices):            # slice sl: the tiles of 64 k from sl * tiles / slices up to (sl + 1) * tiles / slices
            lo, hi = 64 * (sl * (K // 64) // slices), 64 * ((sl + 1) * (K // 64) // slices)
            part = x[:, lo:hi].double() @ w[:, lo:hi].double().T
            assert (y[sl].cpu().double() - part).abs().max() / part.abs().max() < 1e-5, sl
        total = y.cpu().double().sum(0)
        assert (total - ref).abs().max() / ref.abs().max() < 1e-5
        # the norm adds them in order: the same as adding them here
        resid = torch.zeros((M, N), device=DEV)
        ones = torch.ones(N, device=DEV)
        kernels.add_rmsnorm(resid, y, ones, 1e-6, torch.float32)
        acc = torch.zeros((M, N), device=DEV)
        for sl in range(slices):
            acc += y[sl]
        assert torch.equal(resid, acc)
    elif y.dim() == 2:
        assert y.shape == (M, N) and y.dtype == torch.bfloat16
        assert (y.cpu().double() - ref).abs().max() / ref.abs().max() < _tol(torch.bfloat16)
    else:       # the tiled kernel of few rows and its own slices
        assert (y.cpu().double().sum(0) - ref).abs().max() / ref.abs().max() < 1e-5


@pytest.mark.parametrize("shape", [0, 1, 2])
@pytest.mark.parametrize("M,N,K,slices", [(2048, 4096, 4096, 1), (129, 1000, 192, 1), (130, 264, 128, 2), (300, 516, 640, 5),
                                          (1, 4, 64, 1), (257, 260, 3072, 3), (1111, 2560, 9728, 2), (640, 5120, 1024, 4),
                                          (200, 132, 704, 3), (140, 256, 448, 7), (256, 5120, 17408, 6)])
def test_linear_tile_every_shape(M, N, K, slices, shape):
    """The many-row tiled product alone, in its three tile shapes: rows and features that are no
    multiple of a tile (what a tile holds past the end is read from the last row and never
    stored), one slice rounded to bfloat16, several as float32 partial sums; against float64.
    A slice's sum does not depend on the tile shape: the shapes give the same bits."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(43)
    x = _rand((M, K), torch.bfloat16, g)
    w = _rand((N, K), torch.bfloat16, g, scale=0.05)
    ref = x.double() @ w.double().T
    y = kernels.linear_tile(x.to(DEV), w.to(DEV), slices, partial=True, shape=shape)
    assert y.shape == (slices, M, N) and y.dtype == torch.float32
    assert (y.cpu().double().sum(0) - ref).abs().max() / ref.abs().max() < 1e-5
    assert torch.equal(y, kernels.linear_tile(x.to(DEV), w.to(DEV), slices, partial=True, shape=(shape + 1) % 3))
    if slices == 1:
        yb = kernels.linear_tile(x.to(DEV), w.to(DEV), shape=shape)
        assert yb.shape == (M, N) and yb.dtype == torch.bfloat16
        assert torch.equal(yb, y[0].to(torch.bfloat16))          # one rounding of the same float32 sum


def test_linear_tile_refuses():
    from xinfer_amd import kernels
    x = torch.zeros((130, 192), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((64, 192), dtype=torch.bfloat16, device=DEV)
    assert kernels.linear_tile_takes(130, 64, 192, 3) and kernels.linear_tile_takes(130, 64, 192, 2)
    assert not kernels.linear_tile_takes(130, 64, 192, 4)
    with pytest.raises(kernels.KernelError, match="not taken"):
        kernels.linear_tile(x, w, 4, partial=True)                               # more slices than tiles of 64
    with pytest.raises(kernels.KernelError, match="not taken"):
        kernels.linear_tile(x, torch.zeros((66, 192), dtype=torch.bfloat16, device=DEV))      # N no multiple of 4
    with pytest.raises(kernels.KernelError, match="not taken"):
        kernels.linear_tile(x[:, :100].contiguous(), w[:, :100].contiguous())      # K no multiple of 64
    with pytest.raises(kernels.KernelError, match="bfloat16"):
        kernels.linear_tile(x.float(), w.float())
    with pytest.raises(kernels.KernelError, match="shape"):
        kernels.linear_tile(x, w, shape=3)


def test_linear_skinny_plan_fills_the_compute_units():
    """The shapes the streaming product chooses: grids that are multiples of the 256 compute
    units where the width allows (a workgroup may own a number of features that is no multiple
    of 16), slices of K for narrow outputs only when asked, and the same slices for every M."""
    from xinfer_amd import kernels
    for (N, K, gated) in ((4096, 4096, False), (5120, 5120, False), (6144, 4096, False), (5120, 17408, False),
                          (12288, 4096, True)):
        for M in (1, 8, 16):
            ks, rt, rows, wgs = kernels.linear_skinny_plan(M, N, K, gated)
            assert ks == 1 and rows <= 16 * rt // (2 if gated else 1) and wgs % 256 == 0, (N, K, gated, M, rt, rows, wgs)
    assert kernels.linear_skinny_plan(8, 5120, 5120)[2] == 20
    assert kernels.linear_skinny_plan(16, 17408, 5120, gated=True)[3] == 512
    for M in (1, 17, 64):
        assert kernels.linear_skinny_plan(M, 4096, 12288, allow_split=True)[0] == 4
        assert kernels.linear_skinny_plan(M, 151936, 4096, allow_split=True)[0] == 1


def test_linear_skinny_refuses():
    from xinfer_amd import kernels
    x = torch.zeros((65, 64), dtype=torch.bfloat16, device=DEV)
    w = torch.zeros((32, 64), dtype=torch.bfloat16, device=DEV)
    with pytest.raises(kernels.KernelError, match="<= 64"):
        kernels.linear_skinny(x, w)
    with pytest.raises(kernels.KernelError, match="multiple of 8"):
        kernels.linear_skinny(x[:4, :60].contiguous(), w[:, :60].contiguous())
    with pytest.raises(kernels.KernelError, match="bfloat16"):
        kernels.linear_skinny(x[:4].float(), w.float())
    with pytest.raises(kernels.KernelError, match="no kernel of 4 row tiles, 16 waves"):
        kernels.linear_skinny(x[:4].contiguous(), w, row_tiles=4, waves=16)
    with pytest.raises(kernels.KernelError, match="no kernel of 5 row tiles"):
        kernels.linear_skinny(x[:4].contiguous(), w, row_tiles=5, waves=8)
    with pytest.raises(kernels.KernelError, match="no kernel of 8 row tiles"):
        kernels.linear_skinny(x[:40].contiguous(), w, row_tiles=8, waves=8)


def _rope_ref(x, pos, cos, sin, rot, interleaved):
    x = x.double().clone()
    c, s = cos[pos].double()[:, None, :], sin[pos].double()[:, None, :]
    if interleaved:
        a, b = x[..., 0:rot:2].clone(), x[..., 1:rot:2].clone()
        x[..., 0:rot:2], x[..., 1:rot:2] = a * c - b * s, a * s + b * c
    else:
        h = rot // 2
        a, b = x[..., :h].clone(), x[..., h:rot].clone()
        x[..., :h], x[..., h:rot] = a * c - b * s, a * s + b * c
    return x


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,rot,interleaved,norm", [
    (3, 2, 8, 8, False, False),      # the shape of the reference's rope probe (q (11,3,8), k (11,2,8))
    (3, 2, 8, 8, True, False),
    (7, 7, 48, 48, False, True),
    (6, 2, 16, 16, False, True),
    (8, 2, 128, 128, False, True),
    (5, 1, 80, 32, False, True),     # partial rotary
    (4, 2, 256, 256, True, True),
])
def test_qk_norm_rope_kv(dtype, nq, nkv, d, rot, interleaved, norm):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(7)
    # positions of the reference's probe (attention_misc_precision_probe.rs:36-40)
    positions = torch.tensor([0, 7, 2, 31, 9, 16, 3, 63, 4, 12, 5], dtype=torch.int32)
    T, page, pages, eps = positions.numel(), 8, 5, 1e-5
    cos, sin = plain.rope_tables(10000.0, rot, 64)
    qkv = _rand((T, (nq + 2 * nkv) * d), dtype, g)
    qw = (1 + 0.3 * torch.randn(d, generator=g)) if norm else None
    kw = (1 + 0.3 * torch.randn(d, generator=g)) if norm else None
    perm = torch.randperm(pages * page, generator=g)[:T]
    slots = perm.to(torch.int64)
    kc = torch.zeros((pages, nkv, page, d), dtype=dtype)
    vc = torch.zeros_like(kc)
    q_out = kernels.qk_norm_rope_kv(
        qkv.to(DEV), qw.to(DEV) if norm else None, kw.to(DEV) if norm else None, eps, cos.to(DEV),
        sin.to(DEV), rot, interleaved, positions.to(DEV), slots.to(DEV), (kcd := kc.to(DEV)),
        (vcd := vc.to(DEV)), nq, nkv, d)
    x = qkv.double().reshape(T, nq + 2 * nkv, d)
    q, k, v = x[:, :nq], x[:, nq:nq + nkv], x[:, nq + nkv:]
    if norm:
        q, k = plain.rms_norm(q, qw.double(), eps), plain.rms_norm(k, kw.double(), eps)
    q = _rope_ref(q, positions.long(), cos, sin, rot, interleaved)
    k = _rope_ref(k, positions.long(), cos, sin, rot, interleaved)
    tol = _tol(dtype)
    assert (q_out.cpu().double() - q).abs().max() / q.abs().max() < tol
    kcd, vcd = kcd.cpu().double(), vcd.cpu()
    for t in range(T):
        p, o = int(slots[t]) // page, int(slots[t]) % page
        assert (kcd[p, :, o] - k[t]).abs().max() / k.abs().max() < tol, t
        assert torch.equal(vcd[p, :, o].double(), v[t]), t
    # the V pool in groups of eight keys [pages, nkv, page / 8, d, 8] holds the same values
    vt = torch.zeros((pages, nkv, page // 8, d, 8), dtype=dtype, device=DEV)
    q_out_t = kernels.qk_norm_rope_kv(
        qkv.to(DEV), qw.to(DEV) if norm else None, kw.to(DEV) if norm else None, eps, cos.to(DEV),
        sin.to(DEV), rot, interleaved, positions.to(DEV), slots.to(DEV), (kct := kc.to(DEV)), vt, nq, nkv, d,
        v_grouped=True, vector_min_tokens=1)
    assert torch.equal(_ungrouped(vt.cpu()), vcd)
    # q and K of that form (another kernel for bfloat16) against the same reference
    assert (q_out_t.cpu().double() - q).abs().max() / q.abs().max() < tol
    kct = kct.cpu().double()
    for t in range(T):
        p, o = int(slots[t]) // page, int(slots[t]) % page
        assert (kct[p, :, o] - k[t]).abs().max() / k.abs().max() < tol, t
    assert float(kct.permute(0, 2, 1, 3).reshape(pages * page, -1)[~torch.isin(torch.arange(pages * page), slots)].abs().max()) == 0.0
    # nothing but the named slots was written
    touched = torch.zeros(pages * page, dtype=torch.bool)
    touched[slots] = True
    flat = kcd.permute(0, 2, 1, 3).reshape(pages * page, -1)
    assert float(flat[~touched].abs().max()) == 0.0


@pytest.mark.parametrize("nq,nkv,d,rot,interleaved", [(32, 8, 128, 128, False), (6, 3, 48, 32, False), (4, 4, 64, 64, True),
                                                    (10, 2, 80, 80, False)])
def test_qk_norm_rope_kv_many_tokens(nq, nkv, d, rot, interleaved):
    """The bfloat16 form with the V pool in groups of eight keys over several blocks of 64 tokens: runs of
    tokens that follow each other in a page, a block that is not full, and tokens whose slot is
    negative (nothing of theirs may be stored)."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(17)
    T, page, pages, eps = 150, 16, 12, 1e-6
    positions = torch.cat([torch.arange(40, 40 + 100), torch.arange(0, 50)]).to(torch.int32)
    cos, sin = plain.rope_tables(1e6, rot, 256)
    qkv = _rand((T, (nq + 2 * nkv) * d), torch.bfloat16, g)
    qw, kw = 1 + 0.2 * torch.randn(d, generator=g), 1 + 0.2 * torch.randn(d, generator=g)
    page_of = torch.randperm(pages, generator=g)
    slots = torch.cat([page_of[(torch.arange(100) + 8) // page] * page + (torch.arange(100) + 8) % page,
                       page_of[7 + torch.arange(50) // page] * page + torch.arange(50) % page]).to(torch.int64)
    slots[torch.tensor([3, 64, 149])] = -1
    kc = torch.zeros((pages, nkv, page, d), dtype=torch.bfloat16, device=DEV)
    vt = torch.zeros((pages, nkv, page // 8, d, 8), dtype=torch.bfloat16, device=DEV)
    q_out = kernels.qk_norm_rope_kv(qkv.to(DEV), qw.to(DEV), kw.to(DEV), eps, cos.to(DEV), sin.to(DEV), rot,
                                    interleaved, positions.to(DEV), slots.to(DEV), kc, vt, nq, nkv, d,
                                    v_grouped=True)
    x = qkv.double().reshape(T, nq + 2 * nkv, d)
    q = _rope_ref(plain.rms_norm(x[:, :nq], qw.double(), eps), positions.long(), cos, sin, rot, interleaved)
    k = _rope_ref(plain.rms_norm(x[:, nq:nq + nkv], kw.double(), eps), positions.long(), cos, sin, rot, interleaved)
    v = x[:, nq + nkv:]
    tol = _tol(torch.bfloat16)
    assert (q_out.cpu().double() - q).abs().max() / q.abs().max() < tol
    want_k = torch.zeros((pages * page, nkv, d), dtype=torch.float64)
    want_v = torch.zeros((pages * page, nkv, d), dtype=torch.float64)
    keep = slots >= 0
    want_k[slots[keep]] = k[keep]
    want_v[slots[keep]] = v[keep]
    got_k = kc.cpu().double().permute(0, 2, 1, 3).reshape(pages * page, nkv, d)
    got_v = _ungrouped(vt.cpu()).double().permute(0, 2, 1, 3).reshape(pages * page, nkv, d)
    assert (got_k - want_k).abs().max() / k.abs().max() < tol
    assert torch.equal(got_v, want_v)


@pytest.mark.parametrize("dtype,T,nq,nkv,d,rot,interleaved", [
    (torch.float32, 11, 3, 1, 48, 48, False), (torch.bfloat16, 11, 4, 2, 32, 16, True),
    (torch.bfloat16, 150, 5, 5, 48, 48, False), (torch.bfloat16, 150, 2, 1, 128, 64, True)])
def test_qk_norm_rope_kv_bias(dtype, T, nq, nkv, d, rot, interleaved):
    """A bias on the packed projection is added before the norm (q, k) and before the store
    (v), in float32: both kernels (one wave per head; 16 bytes per lane from 128 tokens on)
    against norm(x + b) rotated, and v + b rounded once."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(23)
    page, pages, eps = 8, 24, 1e-5
    positions = torch.randint(0, 200, (T,), generator=g).to(torch.int32)
    cos, sin = plain.rope_tables(10000.0, rot, 200)
    width = (nq + 2 * nkv) * d
    qkv = _rand((T, width), dtype, g)
    bias = torch.randn(width, generator=g) * 0.5
    qw, kw = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    slots = torch.randperm(pages * page, generator=g)[:T].to(torch.int64)
    vt_form = dtype == torch.bfloat16
    kc = torch.zeros((pages, nkv, page, d), dtype=dtype, device=DEV)
    vc = torch.zeros((pages, nkv, page // 8, d, 8) if vt_form else (pages, nkv, page, d), dtype=dtype, device=DEV)
    q_out = kernels.qk_norm_rope_kv(qkv.to(DEV), qw.to(DEV), kw.to(DEV), eps, cos.to(DEV), sin.to(DEV), rot, interleaved,
                                    positions.to(DEV), slots.to(DEV), kc, vc, nq, nkv, d, v_grouped=vt_form,
                                    bias=bias.to(DEV))
    x = (qkv.double() + bias.double()).reshape(T, nq + 2 * nkv, d)
    q = _rope_ref(plain.rms_norm(x[:, :nq], qw.double(), eps), positions.long(), cos, sin, rot, interleaved)
    k = _rope_ref(plain.rms_norm(x[:, nq:nq + nkv], kw.double(), eps), positions.long(), cos, sin, rot, interleaved)
    v = (qkv.float() + bias).to(dtype).reshape(T, nq + 2 * nkv, d)[:, nq + nkv:]
    tol = _tol(dtype)
    assert (q_out.cpu().double() - q).abs().max() / q.abs().max() < tol
    got_k = kc.cpu().double().permute(0, 2, 1, 3).reshape(pages * page, nkv, d)
    got_v = (_ungrouped(vc.cpu()) if vt_form else vc.cpu()).permute(0, 2, 1, 3).reshape(pages * page, nkv, d)
    assert (got_k[slots] - k).abs().max() / k.abs().max() < tol
    assert torch.equal(got_v[slots], v)
    with pytest.raises(kernels.KernelError, match="bias"):
        kernels.qk_norm_rope_kv(qkv.to(DEV), qw.to(DEV), kw.to(DEV), eps, cos.to(DEV), sin.to(DEV), rot, interleaved,
                                positions.to(DEV), slots.to(DEV), kc, vc, nq, nkv, d, v_grouped=vt_form,
                                bias=bias[:-1].contiguous().to(DEV))


@pytest.mark.parametrize("T,nq,nkv,d,rot,interleaved,slices,with_bias", [
    (20, 4, 2, 128, 128, False, 5, False), (33, 6, 3, 48, 32, True, 3, True), (1, 2, 1, 256, 256, False, 1, False),
    (300, 4, 4, 64, 64, False, 8, True)])
def test_qk_norm_rope_kv_of_partial_sums(T, nq, nkv, d, rot, interleaved, slices, with_bias):
    """The packed rows as float32 partial sums of a product cut along K (what the tiled split-K
    product hands on): the kernel adds the slices, then does as with rows; against the plain
    formulas on the sum, and with one wave per head whatever the number of tokens."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(31)
    page, pages, eps = 16, 24, 1e-6
    positions = torch.randint(0, 300, (T,), generator=g).to(torch.int32)
    cos, sin = plain.rope_tables(1e6, rot, 300)
    width = (nq + 2 * nkv) * d
    parts = torch.randn((slices, T, width), generator=g)
    bias = torch.randn(width, generator=g) * 0.5 if with_bias else None
    qw, kw = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    slots = torch.randperm(pages * page, generator=g)[:T].to(torch.int64)
    kc = torch.zeros((pages, nkv, page, d), dtype=torch.bfloat16, device=DEV)
    vc = torch.zeros((pages, nkv, page // 8, d, 8), dtype=torch.bfloat16, device=DEV)
    q_out = kernels.qk_norm_rope_kv(parts.to(DEV), qw.to(DEV), kw.to(DEV), eps, cos.to(DEV), sin.to(DEV), rot, interleaved,
                                    positions.to(DEV), slots.to(DEV), kc, vc, nq, nkv, d, v_grouped=True,
                                    bias=None if bias is None else bias.to(DEV))
    assert q_out.dtype == torch.bfloat16 and tuple(q_out.shape) == (T, nq, d)
    total = parts.double().sum(0) + (0 if bias is None else bias.double())
    x = total.reshape(T, nq + 2 * nkv, d)
    q = _rope_ref(plain.rms_norm(x[:, :nq], qw.double(), eps), positions.long(), cos, sin, rot, interleaved)
    k = _rope_ref(plain.rms_norm(x[:, nq:nq + nkv], kw.double(), eps), positions.long(), cos, sin, rot, interleaved)
    v = x[:, nq + nkv:]
    tol = _tol(torch.bfloat16)
    assert (q_out.cpu().double() - q).abs().max() / q.abs().max() < tol
    got_k = kc.cpu().double().permute(0, 2, 1, 3).reshape(pages * page, nkv, d)
    got_v = _ungrouped(vc.cpu()).double().permute(0, 2, 1, 3).reshape(pages * page, nkv, d)
    assert (got_k[slots] - k).abs().max() / k.abs().max() < tol
    assert (got_v[slots] - v).abs().max() / v.abs().max() < tol
    with pytest.raises(kernels.KernelError, match="partial sums"):
        kernels.qk_norm_rope_kv(parts.to(DEV).to(torch.bfloat16), qw.to(DEV), kw.to(DEV), eps, cos.to(DEV), sin.to(DEV), rot,
                                interleaved, positions.to(DEV), slots.to(DEV), kc, vc, nq, nkv, d, v_grouped=True)


def _paged_case(g, dtype, nq, nkv, d, page, seqs, extra_pages=3):
    """Random K/V of several sequences laid into a paged cache under a shuffled page map.
    `seqs` = list of (context length, number of query tokens at its end)."""
    total_pages = sum(-(-c // page) for c, _ in seqs) + extra_pages
    order = torch.randperm(total_pages, generator=g).tolist()
    kc = torch.zeros((total_pages, nkv, page, d), dtype=dtype)
    vc = torch.zeros_like(kc)
    max_pages = max(-(-c // page) for c, _ in seqs)
    bt = torch.zeros((len(seqs), max_pages), dtype=torch.int32)
    ks, vs, qs, tok_seq, positions = [], [], [], [], []
    for b, (ctx, nq_tok) in enumerate(seqs):
        k = _rand((ctx, nkv, d), dtype, g)
        v = _rand((ctx, nkv, d), dtype, g)
        for lp in range(-(-ctx // page)):
            phys = order.pop()
            bt[b, lp] = phys
            n = min(page, ctx - lp * page)
            kc[phys, :, :n] = k[lp * page:lp * page + n].transpose(0, 1)
            vc[phys, :, :n] = v[lp * page:lp * page + n].transpose(0, 1)
        ks.append(k)
        vs.append(v)
        qs.append(_rand((nq_tok, nq, d), dtype, g))
        tok_seq += [b] * nq_tok
        positions += list(range(ctx - nq_tok, ctx))
    return dict(kc=kc, vc=vc, bt=bt, ks=ks, vs=vs, qs=qs,
                tok_seq=torch.tensor(tok_seq, dtype=torch.int32),
                positions=torch.tensor(positions, dtype=torch.int32))


def _attention_ref(case, seqs, window, scale):
    outs = []
    for b, (ctx, n) in enumerate(seqs):
        k, v = case["ks"][b].double(), case["vs"][b].double()
        q_full = torch.zeros((ctx, case["qs"][b].shape[1], k.shape[2]), dtype=torch.float64)
        q_full[ctx - n:] = case["qs"][b].double()
        o = plain.attention(q_full, k, v, window=window or None, scale=scale)
        outs.append(o[ctx - n:].reshape(n, -1))
    return torch.cat(outs)


ATTN_CASES = [
    # nq, nkv, d, page, window, [(context, queries)]
    (4, 2, 32, 16, 0, [(5, 5), (17, 17), (33, 33)]),
    (6, 2, 16, 8, 0, [(200, 1), (130, 48), (9, 9), (64, 2)]),
    (5, 5, 48, 16, 24, [(100, 100), (31, 1), (24, 24), (25, 2)]),
    (8, 2, 128, 64, 0, [(300, 37), (1, 1), (257, 1)]),
    (3, 1, 80, 4, 7, [(40, 40), (13, 2)]),
    (2, 2, 256, 16, 0, [(70, 70)]),
]


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,d,page,window,seqs", ATTN_CASES)
def test_attention_generic(dtype, nq, nkv, d, page, window, seqs):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(9)
    case = _paged_case(g, dtype, nq, nkv, d, page, seqs)
    scale = 1.0 / math.sqrt(d)
    ref = _attention_ref(case, seqs, window, scale)
    q = torch.cat(case["qs"]).contiguous()
    out = kernels.attention_generic(q.to(DEV), case["kc"].to(DEV), case["vc"].to(DEV), case["bt"].to(DEV),
                                    case["tok_seq"].to(DEV), case["positions"].to(DEV), scale, window)
    err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(dtype, 2), err


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_far_key_stands_out(dtype):
    """One far key among hundreds is made to win the softmax by scaling it and the query:
    a kernel that skips or misplaces it returns a visibly different row."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(11)
    nq, nkv, d, page = 4, 2, 64, 16
    seqs = [(700, 1)]
    case = _paged_case(g, dtype, nq, nkv, d, page, seqs)
    far = 3                                            # position of the key that must win
    qv = case["qs"][0]
    kfar = (qv[0, 0].float() / qv[0, 0].float().norm() * 40).to(dtype)
    case["ks"][0][far, 0] = kfar
    phys, off = int(case["bt"][0, far // page]), far % page
    case["kc"][phys, 0, off] = kfar
    scale = 1.0 / math.sqrt(d)
    ref = _attention_ref(case, seqs, 0, scale)
    assert (ref[0, :d] - case["vs"][0][far, 0].double()).abs().max() < 0.05   # head 0 returns v[far]
    out = kernels.attention_generic(torch.cat(case["qs"]).to(DEV), case["kc"].to(DEV), case["vc"].to(DEV),
                                    case["bt"].to(DEV), case["tok_seq"].to(DEV), case["positions"].to(DEV),
                                    scale, 0)
    err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(dtype, 2), err


# ---- the matrix-core attention kernels (bfloat16, V in groups of eight keys in the cache) -----
def _mfma_inputs(case):
    return (torch.cat(case["qs"]).contiguous().to(DEV), case["kc"].to(DEV), _grouped(case["vc"]).to(DEV), case["bt"].to(DEV))


def _cu_ctx(seqs):
    cu = [0]
    for _, n in seqs:
        cu.append(cu[-1] + n)
    return (torch.tensor(cu, dtype=torch.int32), torch.tensor([c for c, _ in seqs], dtype=torch.int32))


PREFILL_CASES = ATTN_CASES + [
    (8, 2, 128, 64, 0, [(2048, 300), (129, 129), (640, 2)]),     # a cached prefix before the portion
    (8, 2, 128, 16, 0, [(700, 300), (65, 64)]),                  # pages smaller than a tile of 64 keys
    (4, 4, 64, 128, 0, [(1000, 500), (200, 1)]),                 # pages larger than a tile
    (4, 2, 32, 8, 40, [(333, 333)]),                              # head size 32, a window
    (2, 1, 256, 64, 0, [(450, 200)]),                             # head size 256 behind a prefix
    (4, 1, 64, 16, 100, [(500, 260), (99, 99), (101, 3)]),       # window crossing block borders
    (6, 3, 96, 8, 0, [(257, 257)]),
    (2, 1, 16, 8, 5, [(40, 40), (6, 1)]),
    (16, 1, 32, 32, 0, [(77, 33)]),                               # group of 16
]


@pytest.mark.parametrize("nq,nkv,d,page,window,seqs", PREFILL_CASES)
def test_attention_prefill_mfma(nq, nkv, d, page, window, seqs):
    from xinfer_amd import kernels
    if not kernels.mfma_attention_supported(nq, nkv, d, page):
        pytest.skip("the matrix-core kernels need a page of a power of two of at least 8 tokens")
    g = torch.Generator().manual_seed(21)
    case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
    scale = 1.0 / math.sqrt(d)
    ref = _attention_ref(case, seqs, window, scale)
    q, kc, vt, bt = _mfma_inputs(case)
    cu, ctx = _cu_ctx(seqs)
    # every workgroup shape of both kernels: the one whose tiles reach LDS through a ring of direct
    # loads (head sizes 32, 64, 128, 256) and the one that copies them through registers
    for ring in (True, False):
        kernels.PREFILL_RING = ring
        try:
            shapes = (0, 1, 2) if ring and kernels.prefill_ring_supported(d) else (0, 1)
            for small in shapes:
                qb = kernels.prefill_block(d, nq // nkv, small)
                tiles = torch.tensor([(b, q0) for b, (_, n) in enumerate(seqs) for q0 in range(0, n, qb)], dtype=torch.int32)
                out = kernels.attention_prefill_bf16(q, kc, vt, bt, tiles.to(DEV), cu.to(DEV), ctx.to(DEV), scale, window,
                                                     small=small)
                err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
                assert err < _tol(torch.bfloat16, 2), (ring, small, err)
            # the launch order the engine uses: every block once
            rows, small = kernels.prefill_tiles([n for _, n in seqs], [c for c, _ in seqs], d, nq, nkv)
            qb = kernels.prefill_block(d, nq // nkv, small)
            assert sorted(rows) == sorted((b, q0) for b, (_, n) in enumerate(seqs) for q0 in range(0, n, qb))
            out = kernels.attention_prefill_bf16(q, kc, vt, bt, torch.tensor(rows, dtype=torch.int32).to(DEV), cu.to(DEV),
                                                 ctx.to(DEV), scale, window, small=small)
            err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
            assert err < _tol(torch.bfloat16, 2), (ring, err)
        finally:
            kernels.PREFILL_RING = True
    if not kernels.prefill_ring_supported(d):
        with pytest.raises(kernels.KernelError, match="two groups"):
            kernels.attention_prefill_bf16(q, kc, vt, bt, tiles.to(DEV), cu.to(DEV), ctx.to(DEV), scale, window, small=2)
    # the generic kernel reads the grouped pool too
    out2 = kernels.attention_generic(q, kc, vt, bt, case["tok_seq"].to(DEV), case["positions"].to(DEV), scale,
                                     window, v_grouped=True)
    err = (out2.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(torch.bfloat16, 2), err


@pytest.mark.parametrize("d", list(range(16, 257, 16)))
def test_attention_mfma_every_head_size(d):
    """Head sizes in steps of 16 up to 256 through the matrix-core kernels: a portion behind a cached
    prefix and a whole prompt (every workgroup shape), and single tokens (two chunk lengths), with a
    window in one run; three query heads on each of two kv heads."""
    from xinfer_amd import kernels
    nq, nkv, page = 6, 2, 16
    assert kernels.mfma_attention_supported(nq, nkv, d, page)
    scale = 1.0 / math.sqrt(d)
    g = torch.Generator().manual_seed(1000 + d)
    for window in (0, 50):
        seqs = [(230, 90), (70, 70), (1, 1)]
        case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
        ref = _attention_ref(case, seqs, window, scale)
        q, kc, vt, bt = _mfma_inputs(case)
        cu, ctx = _cu_ctx(seqs)
        for small in ((0, 1, 2) if kernels.prefill_ring_supported(d) else (0, 1)):
            qb = kernels.prefill_block(d, nq // nkv, small)
            tiles = torch.tensor([(b, q0) for b, (_, n) in enumerate(seqs) for q0 in range(0, n, qb)], dtype=torch.int32)
            out = kernels.attention_prefill_bf16(q, kc, vt, bt, tiles.to(DEV), cu.to(DEV), ctx.to(DEV), scale, window, small=small)
            err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
            assert err < _tol(torch.bfloat16, 2), ("prefill", window, small, err)
        seqs = [(300, 1), (129, 1), (50, 1), (1, 1)]
        case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
        ref = _attention_ref(case, seqs, window, scale)
        q, kc, vt, bt = _mfma_inputs(case)
        _, ctx = _cu_ctx(seqs)
        if kernels.decode_attention_takes(nq, nkv, d):
            for kpw in (None, 128):
                out = kernels.attention_decode_bf16(q, kc, vt, bt, ctx.to(DEV), 300, scale, window, keys_per_workgroup=kpw)
                err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
                assert err < _tol(torch.bfloat16, 2), ("decode", window, kpw, err)


@pytest.mark.parametrize("nq,nkv,d,page,window", [(8, 2, 64, 16, 0), (5, 5, 48, 16, 24), (32, 8, 128, 64, 0), (10, 2, 128, 64, 0)])
def test_attention_of_a_mixed_batch_splits_between_the_kernels(nq, nkv, d, page, window):
    """A step's attention as the engine asks for it: single tokens of decoding requests at the head of
    the batch go to the decode kernel, the portions behind them to the prefill kernel, into one
    result; with fewer than four at the head, or one of them elsewhere, the prefill kernel takes all."""
    from types import SimpleNamespace
    from xinfer_amd import kernels
    if not kernels.mfma_attention_supported(nq, nkv, d, page):
        pytest.skip("the matrix-core kernels need a page of a power of two of at least 8 tokens")
    scale = 1.0 / math.sqrt(d)
    for seqs, split in (([(300, 1), (77, 1), (1, 1), (1030, 1), (64, 1), (90, 40), (200, 200), (17, 1), (33, 2)], True),
                        ([(300, 1), (77, 1), (90, 40), (64, 1), (31, 1)], False)):
        g = torch.Generator().manual_seed(33)
        case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
        ref = _attention_ref(case, seqs, window, scale)
        q, kc, vt, bt = _mfma_inputs(case)
        cu, cl = _cu_ctx(seqs)
        ctx = SimpleNamespace(block_tables=[bt], ctx_lens=cl.to(DEV), cu_q=cu.to(DEV), max_q_len=max(n for _, n in seqs),
                              max_ctx_len=max(c for c, _ in seqs), num_seqs=len(seqs), cu_q_host=cu.tolist(),
                              ctx_lens_host=cl.tolist(), scratch={}, similar_lengths=False,
                              tok_seq=case["tok_seq"].to(DEV), positions=case["positions"].to(DEV))
        kernels_work = kernels.MIXED_DECODE_WORK
        kernels.MIXED_DECODE_WORK = 1000          # small sizes here: the rule's threshold is for real ones
        try:
            out = kernels.attention(q, kc, vt, ctx, 0, scale, window, v_grouped=True)
        finally:
            kernels.MIXED_DECODE_WORK = kernels_work
        (tiles, small, lead, lead_ctx), = ctx.scratch.values()
        assert (lead, lead_ctx) == ((5, 1030) if split else (0, 0))
        assert sorted(set(tiles[:, 0].tolist())) == [b for b in range(len(seqs)) if b >= lead]
        err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
        assert err < _tol(torch.bfloat16, 2), (split, err)


DECODE_CASES = [
    (4, 2, 32, 16, 0, [(5, 1), (17, 1), (33, 1), (1, 1)]),
    (6, 2, 16, 8, 0, [(200, 1), (130, 1), (513, 1)]),
    (5, 5, 48, 16, 24, [(100, 1), (24, 1), (25, 1), (7, 1)]),
    (32, 8, 128, 64, 0, [(4096, 1), (1, 1), (257, 1), (256, 1), (1025, 1)]),
    (8, 2, 128, 64, 300, [(2000, 1), (299, 1), (301, 1), (600, 1)]),
    (16, 1, 64, 8, 0, [(700, 1)]),
    (2, 2, 256, 16, 0, [(70, 1), (300, 1)]),
]


@pytest.mark.parametrize("nq,nkv,d,page,window,seqs", DECODE_CASES)
def test_attention_decode_mfma(nq, nkv, d, page, window, seqs):
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(22)
    case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
    scale = 1.0 / math.sqrt(d)
    ref = _attention_ref(case, seqs, window, scale)
    q, kc, vt, bt = _mfma_inputs(case)
    _, ctx = _cu_ctx(seqs)
    out = kernels.attention_decode_bf16(q, kc, vt, bt, ctx.to(DEV), int(ctx.max()), scale, window)
    err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(torch.bfloat16, 2), err


@pytest.mark.parametrize("nq,nkv,d,page,window,seqs,kpw", [
    (8, 2, 128, 64, 0, [(7000, 1), (300, 1), (3201, 1)], 256),          # 28 splits, 2 and 13
    (4, 4, 48, 16, 0, [(3300, 1)], 128),                                # 26 splits, a head size of 48
    (2, 1, 256, 16, 0, [(6000, 1), (1, 1)], 128),                       # 47 splits and one
    (6, 2, 64, 32, 4000, [(7000, 1), (3999, 1)], 128),                  # a window over 32 splits
])
def test_attention_decode_many_splits(nq, nkv, d, page, window, seqs, kpw):
    """More than 24 splits go to the sixteen-wave combine kernel: against the plain attention, and
    with one far key made to win the softmax, whose value row must come back."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(29)
    case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
    scale = 1.0 / math.sqrt(d)
    q, kc, vt, bt = _mfma_inputs(case)
    _, ctx = _cu_ctx(seqs)
    longest = int(ctx.max())
    assert (min(longest, window + 31) if window else longest) // kpw + 1 > 24
    ref = _attention_ref(case, seqs, window, scale)
    out = kernels.attention_decode_bf16(q, kc, vt, bt, ctx.to(DEV), longest, scale, window, keys_per_workgroup=kpw)
    err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(torch.bfloat16, 2), err
    far = longest - 1 - (window // 2 if window else longest // 3)       # a key in the middle of the splits
    qv = case["qs"][0]
    gsz = nq // nkv
    for kvh in range(nkv):
        kfar = (qv[0, kvh * gsz].float() / qv[0, kvh * gsz].float().norm() * 80).to(torch.bfloat16)
        case["ks"][0][far, kvh] = kfar
        case["kc"][int(case["bt"][0, far // page]), kvh, far % page] = kfar
    ref = _attention_ref(case, seqs, window, scale)
    assert (ref[0, :d] - case["vs"][0][far, 0].double()).abs().max() < 0.05
    q, kc, vt, bt = _mfma_inputs(case)
    out = kernels.attention_decode_bf16(q, kc, vt, bt, ctx.to(DEV), longest, scale, window, keys_per_workgroup=kpw)
    assert (out.cpu().double() - ref).abs().max() / ref.abs().max() < _tol(torch.bfloat16, 2)


PACKED_CASES = [
    # nq, nkv, d, page, window, rot, interleaved, norm, bias, slices, kpw, contexts
    (32, 8, 128, 64, 0, 128, False, True, False, 0, None, [4096, 1, 257, 256, 1025, 65]),
    (32, 8, 128, 64, 0, 128, False, True, False, 3, 256, [513, 257, 256, 1024, 1]),     # the last position opens a chunk
    (6, 2, 16, 8, 0, 16, False, True, True, 0, 128, [200, 130, 513, 129]),
    (5, 5, 48, 16, 24, 32, False, True, False, 0, None, [100, 24, 25, 7]),              # a window, partial rotation
    (8, 2, 128, 64, 300, 128, True, False, True, 2, 128, [2000, 299, 301, 600]),
    (16, 1, 64, 8, 0, 64, True, True, False, 0, 128, [700, 9]),                         # a group of 16 for four waves
    (2, 2, 256, 16, 0, 256, False, True, True, 5, None, [70, 300]),
    (3, 1, 80, 8, 0, 0, False, False, False, 0, 128, [40, 13, 130]),                    # no rotation, no norm
    (8, 2, 128, 64, 0, 64, False, True, False, 0, 128, [300, 129, 64]),                 # half of the head rotated
    (4, 4, 64, 16, 0, 64, False, True, True, 2, 128, [200, 65, 128]),
    # a window makes chunks start at any multiple of 32: every offset of the last position in its chunk and in
    # its 128-byte line of V^T, among them lines of which the chunk's first reads have already taken a part
    (8, 2, 128, 64, 300, 128, False, True, False, 0, 256, list(range(600, 664))),
    (4, 1, 64, 64, 140, 64, False, True, False, 0, 256, list(range(450, 514))),     # one chunk of 140 to 171 keys
]


@pytest.mark.parametrize("nq,nkv,d,page,window,rot,interleaved,norm,bias,slices,kpw,contexts", PACKED_CASES)
def test_attention_decode_packed_gives_the_bits_of_the_two_kernels(nq, nkv, d, page, window, rot, interleaved, norm,
                                                                   bias, slices, kpw, contexts):
    """A decode step's attention from the packed projection (norm, rotation and cache write inside
    the attention kernel) against the two kernels one after the other: the same output and the same
    cache, bit for bit; a sequence with a negative slot stores nothing; and a new key made to win the
    softmax brings back the new value, so the workgroup that wrote it has read it."""
    from xinfer_amd import kernels
    g = torch.Generator().manual_seed(31)
    seqs = [(c, 1) for c in contexts]
    B, heads = len(seqs), nq + 2 * nkv
    case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
    _, kc, vt, bt = _mfma_inputs(case)
    _, ctx = _cu_ctx(seqs)
    positions = (ctx - 1).to(torch.int32)
    slots = torch.tensor([int(case["bt"][b, (c - 1) // page]) * page + (c - 1) % page for b, c in enumerate(contexts)],
                         dtype=torch.int64)
    slots[B - 1] = -1                     # the last sequence's token is another run's to store
    packed = _rand((B, heads * d), torch.bfloat16, g)
    if slices:
        cut = torch.randn((slices, B, heads * d), generator=g) * 0.3
        cut[0] += packed.float() - cut.sum(0)
        packed = cut
    cos, sin = plain.rope_tables(10000.0, rot, max(contexts) + 1) if rot else (torch.zeros(1, 0), torch.zeros(1, 0))
    qw = (1 + 0.3 * torch.randn(d, generator=g)).to(DEV) if norm else None
    kw = (1 + 0.3 * torch.randn(d, generator=g)).to(DEV) if norm else None
    bs = (0.2 * torch.randn(heads * d, generator=g)).to(DEV) if bias else None
    scale, eps, longest = 1.0 / math.sqrt(d), 1e-5, max(contexts)
    cos, sin, positions, slots, ctx_d = cos.to(DEV), sin.to(DEV), positions.to(DEV), slots.to(DEV), ctx.to(DEV)

    def both(packed):
        k1, v1 = kc.clone(), vt.clone()
        q = kernels.qk_norm_rope_kv(packed.to(DEV), qw, kw, eps, cos, sin, rot, interleaved, positions, slots, k1, v1,
                                    nq, nkv, d, v_grouped=True, vector_min_tokens=1 << 30, bias=bs)
        one = kernels.attention_decode_bf16(q, k1, v1, bt, ctx_d, longest, scale, window, keys_per_workgroup=kpw)
        k2, v2 = kc.clone(), vt.clone()
        two = kernels.attention_decode_packed_bf16(packed.to(DEV), qw, kw, eps, cos, sin, rot, interleaved, positions,
                                                   slots, k2, v2, bt, ctx_d, longest, nq, scale, window, bias=bs,
                                                   keys_per_workgroup=kpw)
        assert torch.equal(k1, k2) and torch.equal(v1, v2)
        assert not torch.equal(k1[:, :, :, :], kc) and not torch.equal(v1, vt)       # something was stored
        assert torch.equal(one, two)
        return two, k2, v2

    out, k2, v2 = both(packed)
    # the sequence with the negative slot: its place in the cache is as it was
    c = contexts[B - 1]
    pg, off = int(case["bt"][B - 1, (c - 1) // page]), (c - 1) % page
    assert torch.equal(k2[pg, :, off], kc[pg, :, off]) and torch.equal(v2[pg, :, off >> 3, :, off & 7], vt[pg, :, off >> 3, :, off & 7])
    if not norm and not rot and not slices:
        # the new key of sequence 0 points along its first query head of every group, far longer than any other
        x = packed.clone().reshape(B, heads, d)
        gsz = nq // nkv
        for kvh in range(nkv):
            qv = x[0, kvh * gsz].float()
            x[0, nq + kvh] = (qv / qv.norm() * 60 / scale / qv.norm()).to(torch.bfloat16)
        out, _, _ = both(x.reshape(B, heads * d))
        new_v = x[0, nq + nkv:].float()
        for kvh in range(nkv):
            assert (out[0].reshape(nq, d)[kvh * gsz].float().cpu() - new_v[kvh]).abs().max() < 0.05, kvh


def test_attention_decode_packed_refuses():
    from xinfer_amd import kernels
    nq, nkv, d, page = 4, 2, 32, 16
    kc = torch.zeros((4, nkv, page, d), dtype=torch.bfloat16, device=DEV)
    vt = torch.zeros((4, nkv, page // 8, d, 8), dtype=torch.bfloat16, device=DEV)
    bt = torch.zeros((2, 2), dtype=torch.int32, device=DEV)
    ctx = torch.tensor([3, 5], dtype=torch.int32, device=DEV)
    pos = (ctx - 1).to(torch.int32)
    slots = torch.tensor([2, 4], dtype=torch.int64, device=DEV)
    cos = torch.ones((8, d // 2), device=DEV)
    good = torch.zeros((2, (nq + 2 * nkv) * d), dtype=torch.bfloat16, device=DEV)

    def call(qkv=good, cos=cos, slots=slots, rot=d, qw=None, kw=None):
        return kernels.attention_decode_packed_bf16(qkv, qw, kw, 1e-6, cos, cos, rot, False, pos, slots, kc, vt, bt, ctx,
                                                    5, nq, 1.0)
    call()
    with pytest.raises(kernels.KernelError, match="is not contiguous"):
        call(qkv=good[:, :-d])
    with pytest.raises(kernels.KernelError, match="bfloat16"):
        call(qkv=good.float())
    with pytest.raises(kernels.KernelError, match="cos/sin"):
        call(rot=d - 2)
    with pytest.raises(kernels.KernelError, match="one block table row"):
        call(slots=slots[:1])
    with pytest.raises(kernels.KernelError, match="both"):
        call(qw=torch.ones(d, device=DEV))


def test_decode_keys_per_workgroup_grow_with_the_work():
    """Sequences of about one length: the splits that make the fewest rounds of workgroups over the
    256 compute units, one round of large chunks where there is one, whole sequences from 256
    (sequence, kv head) pairs on, and workgroups for seven eighths of the units at least where the keys allow.  Mixed
    lengths: chunks of 128 to 512 keys, about 512 workgroups; chunks of 1,024 from one pair a compute unit on, whole
    sequences (up to 2,048 keys) from one and a half."""
    from xinfer_amd import kernels
    plan = lambda pairs, span: kernels.decode_keys_per_workgroup(pairs, span, similar=True)
    assert plan(8, 4096) == 128                  # 32 splits: 256 workgroups
    assert plan(64, 4096) == 1024                # 4 splits: 256 workgroups
    assert plan(128, 8704) == 4352               # 2 splits
    assert plan(96, 4096) == 512                 # 8 splits, three rounds: two splits would leave 64 units idle
    assert plan(8, 8704) == 128                  # 544 small workgroups rather than 184 larger ones
    assert plan(256, 4096) > 4096 and plan(512, 4096) > 4096 and plan(1024, 1 << 20) > 1 << 20      # one split
    assert plan(384, 4096) == 2048               # three rounds of halves, not two of whole sequences
    assert plan(8, 131072) == 4096
    for pairs, span in ((8, 4096), (24, 4096), (40, 3000), (100, 900), (8, 131072)):
        k = plan(pairs, span)
        assert k % 128 == 0 and pairs * -(-span // k) >= 224, (pairs, span, k)
    assert plan(4, 1024) == 128                  # too few keys for 256 workgroups: as many as there are
    mixed = lambda pairs, span: kernels.decode_keys_per_workgroup(pairs, span, similar=False)
    assert mixed(8, 4096) == 128 and mixed(32, 4096) == 256 and mixed(64, 4096) == 512
    assert mixed(200, 2304) == 512 and mixed(8, 131072) == 512
    assert mixed(256, 2304) == 1024 and mixed(512, 2304) == 2048 and mixed(512, 2048) == 2176     # many pairs: longer chunks, whole sequences


@pytest.mark.parametrize("window", [0, 100])
def test_attention_decode_one_split_per_sequence(window):
    """Many sequences of about the same length: a workgroup takes a whole sequence and writes the
    result itself (no partial results, no second kernel).  256 (sequence, kv head) pairs."""
    from xinfer_amd import kernels
    nq, nkv, d, page = 8, 8, 32, 16
    g = torch.Generator().manual_seed(23)
    seqs = [(290 + (7 * b) % 30, 1) for b in range(32)]
    assert kernels.decode_keys_per_workgroup(32 * nkv, 320, similar=True) > 320
    assert kernels.decode_keys_per_workgroup(32 * nkv, 320, similar=False) == 128
    case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
    scale = 1.0 / math.sqrt(d)
    ref = _attention_ref(case, seqs, window, scale)
    q, kc, vt, bt = _mfma_inputs(case)
    _, ctx = _cu_ctx(seqs)
    out = kernels.attention_decode_bf16(q, kc, vt, bt, ctx.to(DEV), int(ctx.max()), scale, window, similar=True)
    err = (out.cpu().double() - ref).abs().max() / ref.abs().max()
    assert err < _tol(torch.bfloat16, 2), err


def test_attention_mfma_far_key_and_page_edges():
    """One key is made to win the softmax, placed in turn at a page's first and last offset,
    at the first key, and just before the query: decode and prefill kernels must return its
    value row; a kernel that drops or misplaces a key returns something else."""
    from xinfer_amd import kernels
    nq, nkv, d, page = 8, 2, 128, 64
    scale = 1.0 / math.sqrt(d)
    for far in (0, 63, 64, 127, 511, 512, 1150, 1198):
        g = torch.Generator().manual_seed(23)
        seqs = [(1200, 1)]
        case = _paged_case(g, torch.bfloat16, nq, nkv, d, page, seqs)
        qv = case["qs"][0]
        for kvh in range(nkv):
            kfar = (qv[0, kvh * 4].float() / qv[0, kvh * 4].float().norm() * 60).to(torch.bfloat16)
            case["ks"][0][far, kvh] = kfar
            phys, off = int(case["bt"][0, far // page]), far % page
            case["kc"][phys, kvh, off] = kfar
        ref = _attention_ref(case, seqs, 0, scale)
        assert (ref[0, :d] - case["vs"][0][far, 0].double()).abs().max() < 0.05
        q, kc, vt, bt = _mfma_inputs(case)
        _, ctx = _cu_ctx(seqs)
        out = kernels.attention_decode_bf16(q, kc, vt, bt, ctx.to(DEV), 1200, scale, 0)
        assert (out.cpu().double() - ref).abs().max() / ref.abs().max() < _tol(torch.bfloat16, 2), far
        cu = torch.tensor([0, 1], dtype=torch.int32)
        tiles = torch.tensor([[0, 0]], dtype=torch.int32)
        for small in (0, 1, 2):
            out = kernels.attention_prefill_bf16(q, kc, vt, bt, tiles.to(DEV), cu.to(DEV), ctx.to(DEV), scale, 0, small=small)
            assert (out.cpu().double() - ref).abs().max() / ref.abs().max() < _tol(torch.bfloat16, 2), (far, small)


# ---- random weights are the same on the CPU and on the GPU ------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_random_weights_do_not_depend_on_the_device(dtype):
    """A linear tensor of [1000, 4096] and a norm tensor, made on the CPU (numpy) and on the GPU
    (the kernel) from the same seed: equal bit for bit, in pieces too."""
    import numpy as np
    from xinfer_amd import kernels
    from xinfer_amd.weights import RandomStore, TensorDecl
    from xinfer_amd.weights.counter_normal import counter_normal
    decls = [TensorDecl("model.layers.3.mlp.down_proj.weight", (1000, 4096)),
             TensorDecl("model.norm.weight", (4096,), "norm"), TensorDecl("b", (77,), "zeros")]
    rs = RandomStore(decls, 11, 0.02, 0.1, dtype)
    for d in decls:
        cpu, gpu = rs.get(d.name, None, "cpu"), rs.get(d.name, None, "cuda:0")
        assert cpu.dtype == gpu.dtype == dtype and cpu.shape == tuple(d.shape)
        assert torch.equal(cpu, gpu.cpu()), d.name
    w = rs.get(decls[0].name, torch.float32, "cuda:0")
    assert abs(float(w.std()) - 0.02) < 2e-4 and abs(float(rs.get("model.norm.weight", torch.float32, "cuda:0").mean()) - 1) < 0.01
    # any piece of the stream, any key
    for key, first, n in [(0, 0, 5000), (2 ** 64 - 1, 123_456_789_012, 4099), (0x9E3779B97F4A7C15, 2 ** 33 + 5, 70_000)]:
        out = torch.empty(n, dtype=torch.float32, device="cuda:0")
        kernels.counter_normal_(out, key, 1.0, 0.0, first=first)
        assert np.array_equal(out.cpu().numpy(), counter_normal(key, first, n)), (key, first, n)
