"""Each HIP kernel alone against its plain PyTorch reference, at sizes other than the
engine's tiny models: head sizes in steps of 16, odd numbers of heads and groups, widths
and vocabularies that are no power of two. float32 compares tightly; bfloat16 compares
with the float32 reference computed from the same bfloat16 inputs."""

import random
from types import SimpleNamespace

import pytest
import torch

from torch_kernels import TorchKernels, uniform_of

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: dict(atol=2e-5, rtol=2e-5), torch.bfloat16: dict(atol=2e-2, rtol=2e-2)}


@pytest.fixture(scope="module")
def kernel_sets():
    from socrates_amd.kernels import HipKernels
    return {dt: (HipKernels(dt, DEV), TorchKernels(dt, DEV)) for dt in DTYPES}


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).to(DEV)


def close(got, want, dtype, **over):
    tol = dict(TOL[dtype], **over)
    torch.testing.assert_close(got.float(), want.float(), **tol)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,V,d", [(1, 7, 16), (5, 331, 72), (33, 1000, 2560)])
def test_embedding(kernel_sets, dtype, N, V, d):
    hip, ref = kernel_sets[dtype]
    table = rnd((V, d), dtype, 1)
    ids = torch.randint(0, V, (N,), dtype=torch.int32, device=DEV)
    got = hip.embedding(ids, table)
    assert got.dtype == torch.float32
    torch.testing.assert_close(got, ref.embedding(ids, table), atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,d,eps", [(1, 64, 1e-6), (7, 72, 1e-5), (19, 2560, 1e-6), (3, 5000, 1e-2), (2, 9000, 1e-6)])
def test_add_rmsnorm(kernel_sets, dtype, N, d, eps):
    hip, ref = kernel_sets[dtype]
    w = (1 + 0.3 * torch.randn(d)).to(DEV)
    res = rnd((N, d), torch.float32, 2, 0.05)          # small rows: eps matters
    delta = rnd((N, d), dtype, 3, 0.05)
    r1, r2 = res.clone(), res.clone()
    close(hip.add_rmsnorm(r1, delta, w, eps), ref.add_rmsnorm(r2, delta, w, eps), dtype)
    torch.testing.assert_close(r1, r2, atol=1e-7, rtol=1e-6)          # the residual was updated
    r1, r2 = res.clone(), res.clone()
    close(hip.add_rmsnorm(r1, None, w, eps), ref.add_rmsnorm(r2, None, w, eps), dtype)
    torch.testing.assert_close(r1, res, atol=0, rtol=0)
    rows = torch.tensor([N - 1, 0, N // 2], dtype=torch.int32, device=DEV)
    r1 = res.clone()
    close(hip.add_rmsnorm(r1, delta, w, eps, rows), ref.add_rmsnorm(res.clone(), delta, w, eps, rows), dtype)
    torch.testing.assert_close(r1, res, atol=0, rtol=0)                # gather mode writes nothing back


@pytest.mark.parametrize("dtype", DTYPES)
def test_rmsnorm_rows_matches_library_routine(kernel_sets, dtype):
    hip, _ = kernel_sets[dtype]
    x = rnd((11, 5, 48), dtype, 4)
    w = (1 + 0.2 * torch.randn(48)).to(DEV)
    want = torch.nn.functional.rms_norm(x.float(), (48,), w, 1e-5)
    close(hip.rmsnorm(x, w, 1e-5), want, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,ff", [(1, 128), (9, 200), (130, 9728)])
def test_swiglu(kernel_sets, dtype, N, ff):
    hip, _ = kernel_sets[dtype]
    gu = rnd((N, 2 * ff), dtype, 5, 2.0)
    want = torch.nn.functional.silu(gu[:, :ff].float()) * gu[:, ff:].float()
    close(hip.swiglu(gu), want, dtype)
    zero_gate = gu.clone()
    zero_gate[:, :ff] = 0
    assert hip.swiglu(zero_gate).abs().max() == 0       # silu is on the gate half
    if ff % 16 == 0:
        # the same with gate and up columns alternating in blocks of 16
        mixed = torch.stack([gu[:, :ff].reshape(N, ff // 16, 16), gu[:, ff:].reshape(N, ff // 16, 16)], 2).reshape(N, 2 * ff)
        close(hip.swiglu(mixed.contiguous(), 16), want, dtype)


@pytest.mark.parametrize("M,ff,K", [(1, 128, 64), (8, 9728, 2560), (16, 160, 96), (5, 48, 256)])
def test_linear_swiglu_fused(kernel_sets, M, ff, K):
    """One kernel for the gate and up products and the activation (rows interleaved by 16)."""
    hip, _ = kernel_sets[torch.bfloat16]
    x = rnd((M, K), torch.bfloat16, 30)
    gate, up = rnd((ff, K), torch.bfloat16, 31, K ** -0.5), rnd((ff, K), torch.bfloat16, 32, K ** -0.5)
    w = torch.stack([gate.view(ff // 16, 16, K), up.view(ff // 16, 16, K)], 1).reshape(2 * ff, K).contiguous()
    want = torch.nn.functional.silu(x.float() @ gate.float().T) * (x.float() @ up.float().T)
    close(hip.linear_swiglu(x, w, 16), want, torch.bfloat16)
    big = rnd((40, K), torch.bfloat16, 33)                # more rows: product, then the activation kernel
    want = torch.nn.functional.silu(big.float() @ gate.float().T) * (big.float() @ up.float().T)
    close(hip.linear_swiglu(big, w, 16), want, torch.bfloat16)


@pytest.mark.parametrize("a_dt,w_dt,c_dt", [
    (torch.float32, torch.float32, torch.float32), (torch.bfloat16, torch.float32, torch.bfloat16),
    (torch.bfloat16, torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16, torch.bfloat16)])
@pytest.mark.parametrize("M,N,K", [(1, 16, 8), (3, 331, 72), (8, 2560, 4096), (17, 100, 200), (33, 257, 96),
                                   (64, 1000, 2560), (65, 130, 264), (130, 384, 96), (300, 700, 1032),
                                   (5, 77, 33)])
def test_linear(kernel_sets, a_dt, w_dt, c_dt, M, N, K):
    hip, _ = kernel_sets[a_dt]
    x, w = rnd((M, K), a_dt, 6), rnd((N, K), w_dt, 7, K ** -0.5)
    want = x.double() @ w.double().T
    for library in (True, False):        # the library product for many rows, and this package's kernels
        hip.library_gemm = library
        got = hip.linear(x, w, out_dtype=c_dt)
        assert got.dtype == c_dt
        if c_dt == torch.float32:
            torch.testing.assert_close(got.double(), want, atol=3e-5, rtol=3e-5)
        else:
            torch.testing.assert_close(got.double(), want, atol=2e-2, rtol=2e-2)
    hip.library_gemm = True


@pytest.mark.parametrize("M,N,K", [(1, 2560, 4096), (8, 2560, 9728), (40, 100, 2048), (64, 6144, 2560)])
def test_linear_split_k_partials(kernel_sets, M, N, K):
    """Narrow outputs spread K over several workgroups and return float32 partial sums that
    the residual-add + norm kernel adds in order."""
    hip, ref = kernel_sets[torch.bfloat16]
    x, w = rnd((M, K), torch.bfloat16, 6), rnd((N, K), torch.bfloat16, 7, K ** -0.5)
    want = x.double() @ w.double().T
    hip.library_gemm = False            # this package's skinny kernel for every M up to 64
    for ks in (0, 1, 2, 4, 7):
        got = hip.linear(x, w, allow_partial=True, k_splits=ks)
        if ks > 1:
            assert got.shape == (ks, M, N) and got.dtype == torch.float32
        total = got.double().sum(0) if got.dim() == 3 else got.double()
        torch.testing.assert_close(total, want, atol=2e-2, rtol=2e-2)
        if got.dim() == 3:
            res = rnd((M, N), torch.float32, 8)
            gain = (1 + 0.1 * torch.randn(N)).to(DEV)
            r1, r2 = res.clone(), res.clone()
            a = hip.add_rmsnorm(r1, got, gain, 1e-6)
            b = ref.add_rmsnorm(r2, got, gain, 1e-6)
            close(a, b, torch.bfloat16)
            torch.testing.assert_close(r1, r2, atol=1e-5, rtol=1e-5)
    hip.library_gemm = True


@pytest.mark.parametrize("M,d,K,eps", [(1, 64, 64, 1e-6), (8, 2560, 4096, 1e-6), (16, 72, 200, 1e-5),
                                       (5, 100, 9728, 1e-2), (5, 104, 9728, 1e-2), (3, 4096, 96, 1e-6), (11, 2560, 9728, 1e-6)])
def test_linear_add_norm_and_products_of_owed_rows(kernel_sets, M, d, K, eps):
    """A projection that adds to the residual stream and leaves the norm's factor to the
    next product (one kernel), against product, sum and norm one after the other: the new
    residual, then the three kinds of product that can consume the rows. Rows are scaled very
    differently, so a factor applied to the wrong row, or left out, shows."""
    from socrates_amd.kernels import NormOwed
    hip, ref = kernel_sets[torch.bfloat16]
    y, w = rnd((M, K), torch.bfloat16, 40), rnd((d, K), torch.bfloat16, 41, K ** -0.5)
    res = rnd((M, d), torch.float32, 42) * torch.logspace(-2, 2, M, device=DEV)[:, None]
    gain = (1 + 0.3 * torch.randn(d)).to(DEV)
    want_res = res.double() + y.double() @ w.double().T
    want_normed = (want_res * torch.rsqrt((want_res ** 2).mean(-1, keepdim=True) + eps) * gain.double())
    if d % 8:
        # no product could take rows owed their norm at this width (they read 8 elements of K at
        # a time): the call gives the normed rows themselves, the residual summed as always
        r = res.clone()
        rows = hip.linear_add_norm(y, w, r, gain, eps)
        assert not isinstance(rows, NormOwed)
        rows = rows.by_rows() if hasattr(rows, "by_rows") else rows
        torch.testing.assert_close(r.double(), want_res, atol=2e-2, rtol=1e-2)
        torch.testing.assert_close(rows.double(), want_normed, atol=2e-2, rtol=2e-2)
        return
    # K split over 2 or 4 workgroups per tile that meet in memory (twice each: the arrival
    # counts must be back at zero after a call); the sums must not depend on who comes last
    hip.addnorm_splits = 1
    r = res.clone()
    first = hip.linear_add_norm(y, w, r, gain, eps)
    for splits in (2, 4, 4, 2):
        hip.addnorm_splits = splits
        r_s = res.clone()
        owed_s = hip.linear_add_norm(y, w, r_s, gain, eps)
        torch.testing.assert_close(r_s, r, atol=2e-3, rtol=1e-4)
        torch.testing.assert_close(owed_s.x, (r_s * gain).to(torch.bfloat16), atol=0, rtol=0)
        again = res.clone()
        hip.linear_add_norm(y, w, again, gain, eps)
        assert torch.equal(again, r_s)
    hip.addnorm_splits = 0
    assert int(hip._split_count.abs().sum()) == 0
    # fewer than 16 weight rows per workgroup (a narrow output over more compute units), from
    # the weights by tile and row by row: the same sums as with 16
    kept = hip.pack_min_elements
    hip.addnorm_splits = 1                       # (K whole, as in `first`: the sums are added in the same order)
    for rows_, pack in ((16, 1), (10, 1), (8, 1 << 40), (13, 1)):
        hip.addnorm_tile_rows, hip.pack_min_elements = rows_, pack
        r_h = res.clone()
        owed_h = hip.linear_add_norm(y, w, r_h, gain, eps)
        assert owed_h.tiles == -(-d // rows_)
        torch.testing.assert_close(r_h, r, atol=0, rtol=0)
        assert torch.equal(owed_h.x, first.x)
        torch.testing.assert_close(owed_h.ssq[:, :owed_h.tiles].sum(-1), first.ssq[:, :first.tiles].sum(-1), rtol=1e-5, atol=1e-6)
    hip.addnorm_tile_rows, hip.pack_min_elements, hip.addnorm_splits = 0, kept, 0
    r = res.clone()
    owed = hip.linear_add_norm(y, w, r, gain, eps)
    tiles = owed.tiles                           # runs of 8 to 16 columns: the weight rows of a workgroup
    assert tiles in {-(-d // h) for h in range(8, 17)} and (M >= 5 or tiles == -(-d // 16))
    assert isinstance(owed, NormOwed) and owed.ssq.shape == (M, (tiles + 3) // 4 * 4)
    torch.testing.assert_close(r.double(), want_res, atol=2e-2, rtol=1e-2)
    torch.testing.assert_close(owed.ssq[:, :tiles].double().sum(-1), (r.double() ** 2).sum(-1), atol=1e-6, rtol=1e-5)
    owed.ssq[:, tiles:] = float("nan")           # the padding is never read
    # the exact values the kernel should have stored, from its own residual
    torch.testing.assert_close(owed.x, (r * gain).to(torch.bfloat16), atol=0, rtol=0)
    normed = (r.double() * torch.rsqrt((r.double() ** 2).mean(-1, keepdim=True) + eps) * gain.double())
    torch.testing.assert_close(normed, want_normed, atol=2e-2, rtol=2e-2)
    # consumers: a plain product, gate / up with the activation, and another projection with a sum
    if True:
        N2 = 331 if d < 1000 else 6144
        w2 = rnd((N2, d), torch.bfloat16, 43, d ** -0.5)
        close(hip.linear(owed, w2), normed @ w2.double().T, torch.bfloat16)
        ff = 160 if d < 1000 else 9728
        gate, up = rnd((ff, d), torch.bfloat16, 44, d ** -0.5), rnd((ff, d), torch.bfloat16, 45, d ** -0.5)
        wgu = torch.stack([gate.view(ff // 16, 16, d), up.view(ff // 16, 16, d)], 1).reshape(2 * ff, d).contiguous()
        want = torch.nn.functional.silu(normed @ gate.double().T) * (normed @ up.double().T)
        close(hip.linear_swiglu(owed, wgu, 16), want, torch.bfloat16)
        w3 = rnd((88, d), torch.bfloat16, 46, d ** -0.5)
        res3 = rnd((M, 88), torch.float32, 47)
        gain3 = (1 + 0.3 * torch.randn(88)).to(DEV)
        r3 = res3.clone()
        owed3 = hip.linear_add_norm(owed, w3, r3, gain3, 1e-5)
        torch.testing.assert_close(r3.double(), res3.double() + normed @ w3.double().T, atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(owed3.x, (r3 * gain3).to(torch.bfloat16), atol=0, rtol=0)
        # a consumer that cannot apply the factor to its sums (a weight kept in float32 because
        # its file stores it so, a float32 result) gets the rows settled (it once stopped with an error)
        close(hip.settle(owed), normed, torch.bfloat16)
        close(hip.linear(owed, w2.float()), normed @ w2.double().T, torch.bfloat16)
        close(hip.linear(owed, w2, out_dtype=torch.float32), normed @ w2.double().T, torch.bfloat16)
        # (three roundings to bfloat16 on this way: the settled rows, the gate and up sums before
        # the activation kernel, the result; bounded against each row's largest value at three
        # times what the products with one rounding are held to, 6e-3)
        act = hip.linear_swiglu(owed, wgu.float(), 16)
        assert ((act.double() - want).abs() / want.abs().amax(-1, keepdim=True)).max() < 1.8e-2
        r4 = res3.clone()
        rows4 = hip.linear_add_norm(owed, w3.float(), r4, gain3, 1e-5)
        torch.testing.assert_close(r4.double(), res3.double() + normed @ w3.double().T, atol=2e-2, rtol=2e-2)
        assert not isinstance(rows4, NormOwed)
    # more than 16 rows, or the switch off: the same call is product, then sum and norm
    hip.fuse_norms = False
    r = res.clone()
    plain = hip.linear_add_norm(y, w, r, gain, eps)
    hip.fuse_norms = True
    assert isinstance(plain, torch.Tensor)
    close(plain, want_normed, torch.bfloat16, atol=3e-2)
    torch.testing.assert_close(r.double(), want_res, atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("M,d,K", [(1, 64, 64), (8, 2560, 4096), (16, 72, 200), (5, 104, 4088), (3, 4096, 96),
                                   (11, 2560, 2568), (7, 330, 1000), (16, 6144, 2560), (4, 48, 8),
                                   (8, 5120, 5120), (16, 208, 4616), (1, 1024, 4104)])
def test_sweep_form_of_the_skinny_products(kernel_sets, M, d, K):
    """The products of at most 16 rows in their sweep form (a workgroup keeps its slices of x
    in registers and walks over the weight tiles), forced on at every size: plain, with
    float32 output, and the two kinds of product that consume rows owed a norm (plain and
    gate / up with the activation), against float64 and against the form of a workgroup per
    tile. Rows are scaled very differently, so a factor applied to the wrong row shows. K
    over 4,096 goes through a wave's registers in two halves; K beyond what a workgroup's
    waves hold that way (5,120) stays with the other form."""
    hip, _ = kernel_sets[torch.bfloat16]
    y, w = rnd((M, K), torch.bfloat16, 50), rnd((d, K), torch.bfloat16, 51, K ** -0.5)
    res = rnd((M, d), torch.float32, 52) * torch.logspace(-2, 2, M, device=DEV)[:, None]
    gain = (1 + 0.3 * torch.randn(d)).to(DEV)
    kept = (hip.sweep_rows, hip.sweep_min_items)
    assert hip._sweep_plan(16, 2560, 9728) is None and hip._sweep_plan(17, 2560, 2560) is None
    assert hip._sweep_plan(8, 19456, 2560, swiglu=True) == (16, 203)

    def run(sweep):
        hip.sweep_rows, hip.sweep_min_items = (1, 1) if sweep else (0, 1)
        assert (hip._sweep_plan(M, d, K) is not None) == sweep
        out = {"plain": hip.linear(y, w), "f32": hip.linear(y, w, out_dtype=torch.float32)}
        r = res.clone()
        owed = hip.linear_add_norm(y, w, r, gain, 1e-6)
        if d % 8 == 0:
            N2 = 331 if d < 1000 else 6144
            w2 = rnd((N2, d), torch.bfloat16, 53, d ** -0.5)
            out["owed_plain"] = hip.linear(owed, w2)
            ff = 160 if d < 1000 else 9728
            wgu = rnd((2 * ff, d), torch.bfloat16, 54, d ** -0.5)
            out["owed_swiglu"] = hip.linear_swiglu(owed, wgu, 16)
            out["swiglu"] = hip.linear_swiglu(owed.x, wgu, 16)
        return out, r

    try:
        got, r = run(True)
        want, _ = run(False)
    finally:
        hip.sweep_rows, hip.sweep_min_items = kept
    exact = y.double() @ w.double().T
    torch.testing.assert_close(got["f32"].double(), exact, atol=3e-5 * max(1, K / 512) ** 0.5, rtol=3e-5)
    close(got["plain"], exact, torch.bfloat16)
    if d % 8 == 0:
        normed = r.double() * torch.rsqrt((r.double() ** 2).mean(-1, keepdim=True) + 1e-6) * gain.double()
        N2 = 331 if d < 1000 else 6144
        close(got["owed_plain"], normed @ rnd((N2, d), torch.bfloat16, 53, d ** -0.5).double().T, torch.bfloat16)
    for name in got:
        # the two forms add K in another order: equal to a rounding of the output type
        tol = dict(atol=1e-4, rtol=1e-4) if got[name].dtype == torch.float32 else dict(atol=2e-2, rtol=2e-2)
        torch.testing.assert_close(got[name].float(), want[name].float(), **tol)


@pytest.mark.parametrize("M,d,K", [(17, 2560, 9728), (64, 2560, 4096), (33, 48, 96), (32, 4096, 12288), (50, 330, 200),
                                   (64, 5120, 25600), (20, 16, 32)])
def test_products_of_17_to_64_rows_with_k_split_over_sweeping_workgroups(kernel_sets, M, d, K):
    """The projection that ends a branch at 17 to 64 rows: partial sums over parts of K, from
    the weights by tile and row by row (the same bits), against float64; then through
    ``linear_add_norm`` against the residual sum and norm in float64. Row m of x is scaled by
    its own factor, so a row that lands in another one's place shows; widths that are no
    multiple of 16 and K that is no multiple of 32 read the rows."""
    hip, _ = kernel_sets[torch.bfloat16]
    y = rnd((M, K), torch.bfloat16, 70) * torch.logspace(-1, 1, M, device=DEV)[:, None].to(torch.bfloat16)
    w = rnd((d, K), torch.bfloat16, 71, K ** -0.5)
    kept = (hip.parts_min_k, hip.pack_min_elements, hip.pack_weights)
    try:
        hip.parts_min_k, hip.pack_min_elements = 32, 1
        plan = hip._parts_plan(M, d, K)
        assert plan is not None and hip._parts_plan(16, d, K) is None and hip._parts_plan(65, d, K) is None
        exact = y.double() @ w.double().T
        got = {}
        for tiles in (True, False):
            hip.pack_weights = tiles
            hip.forget_packed()
            parts = hip.linear(y, w, allow_partial=True)
            assert parts.dtype == torch.float32 and tuple(parts.shape) == (plan[0], M, d)
            assert (hip._by_tile(w)[1] == 1) == (tiles and d % 16 == 0 and K % 32 == 0)
            got[tiles] = parts
            scale = exact.abs().amax(-1, keepdim=True)
            assert ((parts.double().sum(0) - exact).abs() / scale).max() < 2e-5 * max(1, K / 512) ** 0.5
        assert torch.equal(got[True], got[False])
        hip.pack_weights = True
        res = rnd((M, d), torch.float32, 72)
        gain = (1 + 0.3 * torch.randn(d)).to(DEV)
        r = res.clone()
        out = hip.linear_add_norm(y, w, r, gain, 1e-6)
        if type(out).__name__ == "RowsByTile":              # what goes to the next product may lie by tile
            out = out.by_rows()
        h = res.double() + exact
        torch.testing.assert_close(r.double(), h, atol=1e-4 * max(1, K / 512) ** 0.5, rtol=1e-4)
        close(out, h * torch.rsqrt((h ** 2).mean(-1, keepdim=True) + 1e-6) * gain.double(), torch.bfloat16)
        # switched off, the same call goes through the library and agrees to a rounding of its bfloat16 output
        hip.parts_rows, r2 = 0, res.clone()
        try:
            assert hip._parts_plan(M, d, K) is None
            lib_out = hip.linear_add_norm(y, w, r2, gain, 1e-6)
            if type(lib_out).__name__ == "RowsByTile":
                lib_out = lib_out.by_rows()
        finally:
            hip.parts_rows = 64
        torch.testing.assert_close(out.float(), lib_out.float(), atol=3e-2, rtol=3e-2)
    finally:
        hip.parts_min_k, hip.pack_min_elements, hip.pack_weights = kept
        hip.forget_packed()


@pytest.mark.parametrize("M,d,N", [(17, 2560, 6144), (40, 2560, 19456), (64, 4096, 6144), (33, 96, 64), (48, 5120, 640)])
def test_normed_rows_by_tile_into_the_products_with_k_outermost(kernel_sets, M, d, N):
    """The norm before QKV and before gate / up hands 17 to 64 rows over laid out by tile
    ([d / 32, rows rounded up to 16, 32]); the products read them so and give the bits they
    give from rows laid out one after the other."""
    from socrates_amd.kernels import RowsByTile
    hip, _ = kernel_sets[torch.bfloat16]
    res = rnd((M, d), torch.float32, 90)
    delta = rnd((M, d), torch.bfloat16, 91)
    gain = (1 + 0.3 * torch.randn(d)).to(DEV)
    w = rnd((N, d), torch.bfloat16, 92, d ** -0.5)
    kept = hip.stream_min_items
    try:
        hip.stream_min_items = 1
        hip._stream_default = lambda *a, **k: True
        r1, r2 = res.clone(), res.clone()
        tiled = hip.add_rmsnorm(r1, delta, gain, 1e-6, by_tile=True)
        rows = hip.add_rmsnorm(r2, delta, gain, 1e-6)
        assert isinstance(tiled, RowsByTile) and tuple(tiled.data.shape) == (d // 32, (M + 15) // 16 * 16, 32)
        assert torch.equal(tiled.by_rows(), rows) and torch.equal(r1, r2)
        hip.forms.clear()
        assert torch.equal(hip.linear(tiled, w), hip.linear(rows, w))
        assert torch.equal(hip.linear(tiled, w, out_dtype=torch.float32), hip.linear(rows, w, out_dtype=torch.float32))
        assert torch.equal(hip.linear_swiglu(tiled, w, 16), hip.linear_swiglu(rows, w, 16))
        assert hip.forms["stream"] == 4 and hip.forms["stream_swiglu"] == 2, dict(hip.forms)
        # the activation of the gate / up product by tile is the same values, and a projection that
        # ends a branch reads rows by tile in its sweep over parts of K: the same bits
        act_t, act_r = hip.linear_swiglu(tiled, w, 16, by_tile=True), hip.linear_swiglu(rows, w, 16)
        if N % 64 == 0:
            assert isinstance(act_t, RowsByTile) and torch.equal(act_t.by_rows(), act_r)
        kept_k = hip.parts_min_k
        hip.parts_min_k = 32
        try:
            if hip._parts_plan(M, N, d) is not None:
                hip.forms.clear()
                assert torch.equal(hip.linear(tiled, w, allow_partial=True), hip.linear(rows, w, allow_partial=True))
                assert sum(v for k, v in hip.forms.items() if k.startswith("parts_of_k")) == 2, dict(hip.forms)
        finally:
            hip.parts_min_k = kept_k
        # a consumer that wants partial sums, or the library, gets the rows
        parts = hip.linear(tiled, w, allow_partial=True)
        close(parts.sum(0) if parts.dim() == 3 else parts, rows.float() @ w.float().T, torch.bfloat16)
        hip.stream_rows = 0
        assert not isinstance(hip.add_rmsnorm(res.clone(), delta, gain, 1e-6, by_tile=True), RowsByTile)
        close(hip.linear(tiled, w), rows.float() @ w.float().T, torch.bfloat16)
    finally:
        hip.stream_rows, hip.stream_min_items = 64, kept
        del hip._stream_default
    # up to 16 rows, and beyond 64, the norm's output stays as it was
    for n in (16, 65):
        assert not isinstance(hip.add_rmsnorm(rnd((n, d), torch.float32, 93), None, gain, 1e-6, by_tile=True), RowsByTile)


@pytest.mark.parametrize("M,N,K", [(17, 6144, 2560), (64, 6144, 2560), (32, 19456, 2560), (48, 10240, 5120), (33, 330, 200),
                                   (64, 24576, 4096), (20, 16, 32), (64, 40000, 2560), (40, 51200, 5120)])
def test_products_of_17_to_64_rows_with_k_outermost(kernel_sets, M, N, K):
    """QKV, the output head (float32 out) and gate / up with its activation at 17 to 64 rows:
    a workgroup keeps the sums of its tiles in registers and walks over K, against float64
    products; from the weights by tile and row by row (the same bits). Row m of x is scaled by
    its own factor, so a row that lands in another one's place shows; widths that are no
    multiple of 16 and K that is no multiple of 32 read the weights' rows; more tiles than one
    pass of a workgroup holds take several passes."""
    hip, _ = kernel_sets[torch.bfloat16]
    x = rnd((M, K), torch.bfloat16, 80) * torch.logspace(-0.5, 0.5, M, device=DEV)[:, None].to(torch.bfloat16)
    w = rnd((N, K), torch.bfloat16, 81, K ** -0.5)
    kept = (hip.stream_min_items, hip.pack_min_elements, hip.pack_weights)
    try:
        hip.stream_min_items, hip.pack_min_elements = 1, 1
        hip._stream_default = lambda *a, **k: True          # the form under test, whatever its default rule says
        assert hip._stream_plan(M, N, K) is not None and hip._stream_plan(16, N, K) is None and hip._stream_plan(65, N, K) is None
        exact = x.double() @ w.double().T
        scale = exact.abs().amax(-1, keepdim=True)
        bound = 2e-5 * max(1, K / 512) ** 0.5
        got = {}
        for tiles in (True, False):
            hip.pack_weights = tiles
            hip.forget_packed()
            hip.forms.clear()
            out32 = hip.linear(x, w, out_dtype=torch.float32)
            assert hip.forms["stream"] == 1 and out32.dtype == torch.float32, dict(hip.forms)
            assert ((out32.double() - exact).abs() / scale).max() < bound
            out16 = hip.linear(x, w)
            assert torch.equal(out16, out32.to(torch.bfloat16))       # the same sums, rounded once
            got[tiles] = out32
            if N % 32 == 0:
                # rows alternate in blocks of 16: gate rows, then the up rows of the same outputs
                act = hip.linear_swiglu(x, w, 16)
                assert hip.forms["stream_swiglu"] == 1, dict(hip.forms)
                pairs = exact.view(M, N // 32, 2, 16)
                gate, up = pairs[:, :, 0].reshape(M, N // 2), pairs[:, :, 1].reshape(M, N // 2)
                want = torch.nn.functional.silu(gate) * up
                err = (act.double() - want).abs() / want.abs().amax(-1, keepdim=True)
                assert tuple(act.shape) == (M, N // 2) and err.max() < 6e-3        # one rounding to bfloat16
                got[tiles, "act"] = act
        assert torch.equal(got[True], got[False])
        if N % 32 == 0:
            assert torch.equal(got[True, "act"], got[False, "act"])
        # switched off, the same calls go through the library
        hip.stream_rows = 0
        try:
            hip.forms.clear()
            lib = hip.linear(x, w, out_dtype=torch.float32)
            assert hip.forms["stream"] == 0 and hip.forms["library"] == 1
            assert ((lib.double() - exact).abs() / scale).max() < 4 * bound + 1e-4
        finally:
            hip.stream_rows = 64
    finally:
        hip.stream_min_items, hip.pack_min_elements, hip.pack_weights = kept
        del hip._stream_default
        hip.forget_packed()


@pytest.mark.parametrize("M,d,K", [(1, 64, 64), (8, 2560, 4096), (16, 80, 224), (5, 2560, 9728), (3, 4096, 96),
                                   (16, 6144, 2560), (9, 48, 32)])
def test_weights_by_tile_give_the_same_bits(kernel_sets, M, d, K):
    """Products of at most 16 rows read a copy of their weight laid out by tile. The sums are
    added in the same order as from the rows, so every form of product returns the same
    bits either way; a weight changed in place is copied anew; sizes that do not tile, and
    products of more rows, read the rows."""
    hip, _ = kernel_sets[torch.bfloat16]
    y, w = rnd((M, K), torch.bfloat16, 60), rnd((d, K), torch.bfloat16, 61, K ** -0.5)
    res = rnd((M, d), torch.float32, 62)
    gain = (1 + 0.3 * torch.randn(d)).to(DEV)
    w2 = rnd((6144 if d > 1000 else 336, d), torch.bfloat16, 63, d ** -0.5)
    ff = 9728 if d > 1000 else 160
    wgu = rnd((2 * ff, d), torch.bfloat16, 64, d ** -0.5)
    kept = (hip.pack_weights, hip.pack_min_elements, hip.sweep_rows, hip.sweep_min_items, hip.addnorm_splits)

    def run(pack, sweep, splits):
        hip.pack_weights, hip.pack_min_elements = pack, 0
        hip.sweep_rows, hip.sweep_min_items = (1, 1) if sweep else (0, 1)
        hip.addnorm_splits = splits
        hip.forget_packed()
        out = [hip.linear(y, w), hip.linear(y, w, out_dtype=torch.float32)]
        r = res.clone()
        owed = hip.linear_add_norm(y, w, r, gain, 1e-6)
        out += [r, owed.x, owed.ssq[:, :(d + 15) // 16].clone()]
        if d % 32 == 0:
            out += [hip.linear(owed, w2), hip.linear_swiglu(owed, wgu, 16), hip.linear_swiglu(owed.x, wgu, 16)]
            # what the gate / up product hands on may lie by tile; the projection that takes it
            # returns the same bits as from rows, and so does any other consumer
            act = hip.linear_swiglu(owed, wgu, 16, by_tile=True)
            assert type(act).__name__ == "RowsByTile" and act.shape == (M, ff)
            assert torch.equal(act.by_rows(), out[-2])
            w4 = rnd((d, ff), torch.bfloat16, 66, ff ** -0.5)
            r_rows, r_tile = res.clone(), res.clone()
            o_rows = hip.linear_add_norm(act.by_rows(), w4, r_rows, gain, 1e-6)
            o_tile = hip.linear_add_norm(act, w4, r_tile, gain, 1e-6)
            assert torch.equal(r_rows, r_tile) and torch.equal(o_rows.x, o_tile.x) and torch.equal(o_rows.ssq, o_tile.ssq)
            assert torch.equal(hip.linear(act, w4), hip.linear(act.by_rows(), w4))
            out += [r_tile, o_tile.x]
        assert bool(hip._packed) == pack
        return out

    try:
        for sweep in (False, True):
            for splits in (1, 2):
                by_row, by_tile = run(False, sweep, splits), run(True, sweep, splits)
                for a, b in zip(by_row, by_tile):
                    assert torch.equal(a, b)
        before = hip.linear(y, w)
        w.mul_(2)
        assert torch.equal(hip.linear(y, w).float(), 2 * before.float())         # the copy followed the weight
        odd = rnd((d + 8, K), torch.bfloat16, 65)
        assert hip._by_tile(odd)[1] == 0 and hip._by_tile(odd[:d])[1] == 1
    finally:
        hip.pack_weights, hip.pack_min_elements, hip.sweep_rows, hip.sweep_min_items, hip.addnorm_splits = kept
        hip.forget_packed()


def test_linear_float32_is_not_reduced_precision(kernel_sets):
    """Values that bfloat16 or a 19-bit matrix mode would round away survive."""
    hip, _ = kernel_sets[torch.float32]
    x = torch.full((4, 64), 1.0 + 2.0 ** -20, device=DEV)
    w = torch.full((8, 64), 1.0 + 2.0 ** -20, device=DEV)
    got = hip.linear(x, w)
    want = 64 * (1.0 + 2.0 ** -20) ** 2
    assert abs(got[0, 0].item() - want) < 1e-4 and abs(got[0, 0].item() - 64.0) > 5e-5


def make_paged_case(lens, Hq, Hkv, D, bs, dtype, seed, width=None, spare=5):
    """Random K/V scattered over shuffled pages, one cache row per sequence, with the
    contiguous K/V of each row for the reference."""
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    need = sum(-(-n // bs) for n in lens)
    pages = list(range(1, need + spare + 1))
    rng.shuffle(pages)
    width = width or max(-(-n // bs) for n in lens) + 1
    k_pool = torch.randn(need + spare + 1, Hkv, bs, D, generator=g)
    v_pool = torch.randn(need + spare + 1, Hkv, bs, D, generator=g)
    table = torch.zeros(len(lens), width, dtype=torch.int32)
    dense = []
    for r, n in enumerate(lens):
        nb = -(-n // bs)
        mine = [pages.pop() for _ in range(nb)]
        table[r, :nb] = torch.tensor(mine, dtype=torch.int32)
        k = k_pool[mine].permute(1, 0, 2, 3).reshape(Hkv, nb * bs, D)[:, :n]
        v = v_pool[mine].permute(1, 0, 2, 3).reshape(Hkv, nb * bs, D)[:, :n]
        dense.append((k.to(dtype).float(), v.to(dtype).float()))
    slot = SimpleNamespace(k=k_pool.to(dtype).to(DEV), v=v_pool.to(dtype).to(DEV),
                           block_table=table.to(DEV), block_size=bs, window=None)
    return slot, dense


def ctx_for(token_rows, positions):
    """Device arrays plus the host view of the sequences: a sequence is a run of tokens of
    one row at consecutive positions."""
    import numpy as np
    starts = [0] + [t for t in range(1, len(positions))
                    if token_rows[t] != token_rows[t - 1] or positions[t] != positions[t - 1] + 1]
    qstart = np.array(starts + [len(positions)], dtype=np.int32)
    return SimpleNamespace(positions=torch.tensor(positions, dtype=torch.int32, device=DEV),
                           token_rows=torch.tensor(token_rows, dtype=torch.int32, device=DEV),
                           max_ctx_len=max(positions) + 1, max_q_len=int(np.diff(qstart).max()),
                           host={"seq_qstart": qstart})


def dense_attention(q, dense, token_rows, positions, scale, window=None):
    """Per token: plain softmax attention over the row's contiguous keys lo..p."""
    N, Hq, D = q.shape
    out = torch.empty(N, Hq * D)
    for t in range(N):
        k, v = dense[token_rows[t]]
        p = positions[t]
        lo = 0 if window is None else max(0, p - window + 1)
        k, v = k[:, lo:p + 1], v[:, lo:p + 1]
        G = Hq // k.shape[0]
        o = torch.nn.functional.scaled_dot_product_attention(
            q[t].float().cpu().view(k.shape[0], G, 1, D), k[:, None], v[:, None], scale=scale)
        out[t] = o.reshape(Hq * D)
    return out


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,bs", [(4, 2, 16, 16), (8, 2, 32, 8), (6, 2, 48, 16), (5, 5, 80, 4),
                                         (32, 8, 128, 16), (16, 1, 64, 32), (2, 1, 256, 16)])
def test_paged_attention_decode_tokens(kernel_sets, dtype, Hq, Hkv, D, bs):
    hip, _ = kernel_sets[dtype]
    lens = [1, 15, 16, 17, 300, 1025]
    slot, dense = make_paged_case(lens, Hq, Hkv, D, bs, dtype, seed=D)
    rows, pos = list(range(len(lens))), [n - 1 for n in lens]
    q = rnd((len(lens), Hq, D), dtype, 8)
    want = dense_attention(q, dense, rows, pos, 0.3)
    for splits in (None, (128, 9), (64, 17), (1 << 30, 1)):
        hip.attention_splits = splits
        got = hip.paged_attention(q, slot, ctx_for(rows, pos), 0.3)
        close(got.cpu(), want, dtype, atol=3e-5 if dtype == torch.float32 else 2e-2)
    hip.attention_splits = None


@pytest.mark.parametrize("D,bs", [(256, 24), (256, 8), (256, 12), (192, 24), (160, 4), (128, 24)])
def test_attention_walks_of_large_heads_over_pages_of_any_size(kernel_sets, D, bs):
    """Head sizes above 128 with pages that hold no multiple of 16 keys (every lane looks its own
    key's page up), walks long enough for the loop over rounds of three tiles, with one split and
    with several, a decoded token and a portion; a large scale, so that a key read from the
    wrong place shows (a reordering of this kernel's first loads once gave wrong sums in just
    this corner, and nothing in the tests came near it)."""
    hip, _ = kernel_sets[torch.bfloat16]
    lens = [1116, 100, 203]
    slot, dense = make_paged_case(lens, 8, 2, D, bs, torch.bfloat16, seed=D + bs)
    rows = [0] * 4 + [1] + [2] * 3
    pos = list(range(1112, 1116)) + [99] + list(range(200, 203))
    q = rnd((len(rows), 8, D), torch.bfloat16, 5)
    want = dense_attention(q, dense, rows, pos, 0.3)
    for splits in (None, (1 << 30, 1), (256, 8), (128, 12)):
        hip.attention_splits = splits
        got = hip.paged_attention(q, slot, ctx_for(rows, pos), 0.3)
        close(got.cpu(), want, torch.bfloat16, atol=3e-2)
    hip.attention_splits = None


@pytest.mark.parametrize("Hq,Hkv,D,bs,norm,rope", [(32, 8, 128, 16, True, True), (16, 1, 64, 32, True, True),
                                                   (8, 2, 32, 8, True, False), (6, 3, 128, 4, False, True),
                                                   (2, 1, 256, 16, True, True), (40, 2, 64, 12, False, False),
                                                   (5, 5, 96, 2, True, False)])
def test_decode_attention_from_raw_qkv(kernel_sets, Hq, Hkv, D, bs, norm, rope):
    """A decode step's attention in one kernel (per-head norm, rotation, the new key and value,
    the walk over the pages) against the kernels one after the other, and against plain
    attention on what those wrote: lengths at page and tile edges (a first token, a new page,
    a full tile), with and without key splits, window, norm and rotation. The page slot of the
    new token holds poison before the call and the new key and value after it."""
    hip, _ = kernel_sets[torch.bfloat16]
    lens = [1, 15, 16, 17, 33, 300, 1025]
    N = len(lens)
    rows, pos = list(range(N)), [n - 1 for n in lens]
    q_gain = (1 + 0.3 * torch.randn(D)).to(DEV) if norm else None
    k_gain = (1 + 0.3 * torch.randn(D)).to(DEV) if norm else None
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV) if rope else None
    qkv = rnd((N, (Hq + 2 * Hkv) * D), torch.bfloat16, 60, 1.5)
    ctx = ctx_for(rows, pos)
    table = None
    if rope:
        # the table in two pieces, as a part grows it; it holds what an accurate sincosf gives
        table = torch.empty((1100, 2, D // 2), dtype=torch.float32, device=DEV)
        hip.rope_table(inv_freq, 0, 300, table[:300])
        hip.rope_table(inv_freq, 300, 800, table[300:])
        ang = torch.arange(1100, dtype=torch.float32)[:, None] * inv_freq.cpu()[None]
        torch.testing.assert_close(table[:, 0].cpu(), ang.double().cos().float(), atol=2e-6, rtol=0)
        torch.testing.assert_close(table[:, 1].cpu(), ang.double().sin().float(), atol=2e-6, rtol=0)
    for window in (None, 40):
        for splits in (None, (64, 17), (16, 256), (1 << 30, 1)):
            hip.attention_splits = splits
            slot_a, _ = make_paged_case(lens, Hq, Hkv, D, bs, torch.bfloat16, seed=D + 2)
            slot_b, _ = make_paged_case(lens, Hq, Hkv, D, bs, torch.bfloat16, seed=D + 2)
            for slot in (slot_a, slot_b):               # poison where the new tokens go
                for r, p_ in zip(rows, pos):
                    page = int(slot.block_table[r, p_ // bs])
                    slot.k[page, :, p_ % bs] = float("nan")
                    slot.v[page, :, p_ % bs] = float("inf")
            hip.fuse_rope = False
            q = hip.qk_norm_rope_write(qkv, Hq, Hkv, D, q_gain, k_gain, 1e-6, inv_freq, D if rope else 0,
                                       ctx.positions, ctx.token_rows, slot_a)
            want = hip.paged_attention(q, slot_a, ctx, 0.2, window)
            hip.fuse_rope = True
            got = hip.decode_attention(qkv, Hq, Hkv, D, q_gain, k_gain, 1e-6, table, slot_b, ctx, 0.2, window, True)
            assert got is not None and hip.last_attention_kernel == ("fused", 1)
            close(got, want, torch.bfloat16)
            # the pages: values exact, keys to a rounding of bfloat16 (the sum of squares is added in another order)
            assert torch.equal(slot_b.v, slot_a.v)
            torch.testing.assert_close(slot_b.k.float(), slot_a.k.float(), atol=2e-2, rtol=1e-2)
            # reading only (another layer wrote the slot): queries from a row without k and v heads
            got_r = hip.decode_attention(qkv[:, :Hq * D].contiguous(), Hq, Hkv, D, q_gain, k_gain, 1e-6, table,
                                         slot_a, ctx, 0.2, window, False)
            close(got_r, want, torch.bfloat16)
            # the output laid out by tile for the projection behind it: the same bits
            tiled = hip.decode_attention(qkv[:, :Hq * D].contiguous(), Hq, Hkv, D, q_gain, k_gain, 1e-6, table,
                                         slot_a, ctx, 0.2, window, False, by_tile=True)
            if (Hq * D) % 32 == 0:
                assert type(tiled).__name__ == "RowsByTile" and tiled.shape == (N, Hq * D)
                assert tiled.data.shape[1] == (N + 15) // 16 * 16
                assert torch.equal(tiled.by_rows(), got_r)
            else:
                assert torch.equal(tiled, got_r)
    hip.attention_splits = None
    assert int(hip._split_count.abs().sum()) == 0
    # where the form does not apply the caller is told so
    assert hip.decode_attention(qkv[:, :(Hq + 2 * Hkv) * 16], Hq, Hkv, 16, None, None, 1e-6, None, slot_a, ctx, 0.2) is None
    table32 = torch.zeros((1100, 2, 16), device=DEV)      # a rotation at head size 32: partners lie in different lanes
    assert hip.decode_attention(qkv[:, :(Hq + 2 * Hkv) * 32], Hq, Hkv, 32, None, None, 1e-6, table32, slot_a, ctx, 0.2) is None


def plain_norm_rotate(x, gain, eps, positions, inv_freq):
    """Per-head RMSNorm (x / sqrt(mean(x^2) + eps) * gain) and the rotate-half rotation of
    x [N, H, D] in float32 on the CPU, rounded to bfloat16 once as a kernel's output is."""
    x = x.float().cpu()
    if gain is not None:
        x = x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps) * gain.cpu()
    if inv_freq is not None:
        ang = torch.tensor(positions, dtype=torch.float32)[:, None] * inv_freq.cpu()[None]
        cos, sin = torch.cat([ang.cos()] * 2, -1)[:, None], torch.cat([ang.sin()] * 2, -1)[:, None]
        h = x.shape[-1] // 2
        x = x * cos + torch.cat([-x[..., h:], x[..., :h]], -1) * sin
    return x.to(torch.bfloat16).float()


@pytest.mark.parametrize("Hq,Hkv,D,bs,rope", [(32, 8, 128, 16, True), (16, 1, 64, 32, True), (12, 3, 96, 8, False),
                                              (6, 2, 128, 4, True)])
@pytest.mark.parametrize("window", [None, 1, 16, 17, 40])
def test_decode_attention_against_plain_attention(kernel_sets, Hq, Hkv, D, bs, rope, window):
    """The one-kernel decode attention against plain float32 attention (norm, rotation and
    softmax written out here, contiguous keys): lengths on both sides of a 16-key tile, of a
    page and of the window; with and without key splits. For every row one early key is made
    to win the softmax of one query head: the last key that the window hides (it must change
    nothing) or, in a second pass, the first that it shows (the output is that key's value)."""
    hip, _ = kernel_sets[torch.bfloat16]
    lens = [1, 15, 16, 17, 18, 33, 41, 48, 49, 300, 1025]
    N, G, scale, eps = len(lens), Hq // Hkv, 0.2, 1e-6
    rows, pos = list(range(N)), [n - 1 for n in lens]
    g = torch.Generator().manual_seed(D + (window or 0))
    q_gain = (1 + 0.3 * torch.randn(D, generator=g)).to(DEV)
    k_gain = (1 + 0.3 * torch.randn(D, generator=g)).to(DEV)
    inv_freq = (1.0 / (10000.0 ** (torch.arange(0, D, 2).float() / D))).to(DEV) if rope else None
    table = hip.rope_table(inv_freq, 0, 1100) if rope else None
    qkv = rnd((N, (Hq + 2 * Hkv) * D), torch.bfloat16, 61, 1.5)
    heads = qkv.view(N, Hq + 2 * Hkv, D)
    q = plain_norm_rotate(heads[:, :Hq], q_gain, eps, pos, inv_freq)
    k_new = plain_norm_rotate(heads[:, Hq:Hq + Hkv], k_gain, eps, pos, inv_freq)
    v_new = heads[:, Hq + Hkv:].float().cpu()
    ctx = ctx_for(rows, pos)
    for needle in ("hidden", "shown"):
        slot, dense = make_paged_case(lens, Hq, Hkv, D, bs, torch.bfloat16, seed=D + 3)
        planted = {}
        for r, n in enumerate(lens):
            k, v = dense[r]
            k[:, n - 1], v[:, n - 1] = k_new[r], v_new[r]              # the token's own key and value
            first = 0 if window is None else max(0, n - window)        # the first key the token sees
            j = first - 1 if needle == "hidden" else first
            if j < 0 or j >= n - 1:
                continue                                               # (the token's own key comes from qkv)
            h = (r % Hkv) * G                                          # a query head of kv head r % Hkv
            key = (q[r, h] * (30.0 / (scale * float(q[r, h].pow(2).sum())))).to(torch.bfloat16)
            k[r % Hkv, j] = key.float()
            slot.k[int(slot.block_table[r, j // bs]), r % Hkv, j % bs] = key.to(DEV)
            planted[r] = (h, j)
        want = dense_attention(q.to(torch.bfloat16), dense, rows, pos, scale, window)
        if needle == "shown":
            for r, (h, j) in planted.items():                          # the oracle itself saw the needle
                assert (want[r].view(Hq, D)[h] - dense[r][1][r % Hkv, j]).abs().max() < 0.02
        for splits in (None, (16, 68), (64, 17), (1 << 30, 1)):
            hip.attention_splits = splits
            pages = (slot.k.clone(), slot.v.clone())
            got = hip.decode_attention(qkv, Hq, Hkv, D, q_gain, k_gain, eps, table, slot, ctx, scale, window, True)
            assert got is not None
            close(got.cpu(), want, torch.bfloat16)
            slot.k.copy_(pages[0]), slot.v.copy_(pages[1])
        hip.attention_splits = None
        if window not in (None, 1):
            assert len(planted) >= 5            # rows long enough to have a key on that side of the window's edge
    hip.attention_splits = (16, 8)              # splits that do not reach the longest row's last key are refused
    with pytest.raises(Exception, match="do not cover"):
        hip.decode_attention(qkv, Hq, Hkv, D, q_gain, k_gain, eps, table, slot, ctx, scale, window, True)
    hip.attention_splits = None
    assert int(hip._split_count.abs().sum()) == 0


def test_workgroups_that_meet_in_memory_give_the_same_bits_every_time(kernel_sets):
    """The decode attention with more than four key splits and the projection with the
    residual epilogue whose K is shared by four workgroups exchange partial results through
    memory inside one launch, ordered by an arrival count and no fence. A partial result read
    before it had arrived would change the sum: the same launch, repeated a few hundred times
    on one input, has to give the same bits every time and leave the counts at zero. Stops at
    the first difference."""
    hip, _ = kernel_sets[torch.bfloat16]
    # attention: 8 rows of 8 kv heads, 2,048 keys each, 16 splits (the benchmark's decode step)
    Hq, Hkv, D, bs, N = 32, 8, 128, 16, 8
    lens = [2048 - 37 * r for r in range(N)]
    slot, _ = make_paged_case(lens, Hq, Hkv, D, bs, torch.bfloat16, seed=4)
    rows, pos = list(range(N)), [n - 1 for n in lens]
    ctx = ctx_for(rows, pos)
    qkv = rnd((N, (Hq + 2 * Hkv) * D), torch.bfloat16, 62)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, D, 2).float() / D))).to(DEV)
    table = hip.rope_table(inv_freq, 0, 2048)
    gain = torch.ones(D, device=DEV)
    hip.forms.clear()
    first = None
    for i in range(300):
        got = hip.decode_attention(qkv, Hq, Hkv, D, gain, gain, 1e-6, table, slot, ctx, D ** -0.5, None, True)
        if first is None:
            first = got.clone()
            assert max(int(k.split(":")[1]) for k in hip.forms if k.startswith("fused_attention")) > 4
        elif not torch.equal(got, first):
            raise AssertionError(f"decode attention, launch {i}: {int((got != first).sum())} values differ from the first launch")
    assert int(hip._split_count.abs().sum()) == 0
    # the down projection of a 32B-sized layer at 8 rows: four workgroups per tile of 16 outputs
    M, Nout, K = 8, 5120, 25600
    y, w = rnd((M, K), torch.bfloat16, 63, 0.5), rnd((Nout, K), torch.bfloat16, 64, 0.02)
    norm_gain = (1 + 0.1 * torch.randn(Nout)).to(DEV)
    residual = rnd((M, Nout), torch.float32, 65)
    hip.forms.clear()
    first = None
    for i in range(200):
        res = residual.clone()
        owed = hip.linear_add_norm(y, w, res, norm_gain, 1e-6)
        if first is None:
            first = (owed.x.clone(), owed.ssq.clone(), res.clone())
            assert hip.forms["add_norm:4"] == 1, dict(hip.forms)
        elif not (torch.equal(owed.x, first[0]) and torch.equal(owed.ssq, first[1]) and torch.equal(res, first[2])):
            raise AssertionError(f"linear_add_norm, launch {i}: the result differs from the first launch")
    assert int(hip._split_count.abs().sum()) == 0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,bs", [(8, 2, 64, 16), (6, 3, 48, 4), (32, 8, 128, 16)])
def test_attention_with_further_score_terms(kernel_sets, dtype, Hq, Hkv, D, bs):
    """A bias by distance, a soft cap and a sink logit per head, one at a time and together,
    with and without key splits and a window, decoded tokens and a prompt portion, in both
    dtypes (such a layer goes to the kernel that computes scores on the vector units), against
    the torch stand-in's formulas on the same pages; also a scale that is not positive."""
    hip, ref = kernel_sets[dtype]
    lens = [1, 17, 70, 300]
    slot, _ = make_paged_case(lens, Hq, Hkv, D, bs, dtype, seed=D + 7)
    rows = [0, 1] + [2] * 20 + [3]
    pos = [0, 16] + list(range(50, 70)) + [299]
    q = rnd((len(rows), Hq, D), dtype, 31)
    ctx = ctx_for(rows, pos)
    sinks = torch.linspace(-2, 3, Hq, device=DEV)
    slopes = -torch.logspace(-3, -0.5, Hq, device=DEV)
    cases = [dict(softcap=4.0), dict(sinks=sinks), dict(slopes=slopes), dict(softcap=2.5, sinks=sinks, slopes=slopes)]
    for terms in cases:
        for window in (None, 33):
            want = ref.paged_attention(q, slot, ctx, 0.3, window, terms=terms)
            for splits in (None, (64, 5), (1 << 30, 1)):
                hip.attention_splits = splits
                got = hip.paged_attention(q, slot, ctx, 0.3, window, terms=terms)
                close(got.cpu(), want.cpu(), dtype, atol=3e-5 if dtype == torch.float32 else 2e-2)
            hip.attention_splits = None
        plain_ = ref.paged_attention(q, slot, ctx, 0.3, None)
        assert (ref.paged_attention(q, slot, ctx, 0.3, None, terms=terms).float() - plain_.float()).abs().max() > 0.02
    got = hip.paged_attention(q, slot, ctx, -0.2)              # the MFMA kernels want a positive scale
    close(got.cpu(), ref.paged_attention(q, slot, ctx, -0.2, None).cpu(), dtype, atol=3e-5 if dtype == torch.float32 else 2e-2)
    with pytest.raises(Exception, match="unknown score terms"):
        hip.paged_attention(q, slot, ctx, 0.3, terms=dict(alibi=slopes))


@pytest.mark.parametrize("dtype", DTYPES)
def test_paged_attention_prompt_portions_and_window(kernel_sets, dtype):
    """Tokens of one row at consecutive positions (a portion that starts mid-sequence)
    beside single tokens of other rows, with and without a window."""
    hip, _ = kernel_sets[dtype]
    Hq, Hkv, D, bs = 6, 2, 32, 8
    lens = [70, 9, 130]
    slot, dense = make_paged_case(lens, Hq, Hkv, D, bs, dtype, seed=11)
    rows = [0] * 30 + [1] + [2] * 5
    pos = list(range(40, 70)) + [8] + list(range(125, 130))
    q = rnd((len(rows), Hq, D), dtype, 9)
    for window in (None, 1, 7, 16, 64):
        want = dense_attention(q, dense, rows, pos, D ** -0.5, window)
        # (row tiles, splits, workgroup kernel): the per-wave and the workgroup MFMA kernels
        for row_tiles, splits, wg in ((None, None, True), (1, None, True), (2, None, True), (32, None, True), (64, None, True), (1, (32, 5), False),
                                      (2, None, False), (4, (64, 3), False), (4, None, False)):
            hip.attention_row_tiles, hip.attention_splits, hip.attention_workgroup = row_tiles, splits, wg
            got = hip.paged_attention(q, slot, ctx_for(rows, pos), D ** -0.5, window)
            close(got.cpu(), want, dtype, atol=3e-5 if dtype == torch.float32 else 2e-2)
    hip.attention_row_tiles = hip.attention_splits = None
    hip.attention_workgroup = True


@pytest.mark.parametrize("Hq,Hkv,D,bs", [(4, 2, 16, 16), (9, 3, 48, 4), (32, 8, 128, 16), (16, 1, 64, 32), (40, 2, 32, 8),
                                         (8, 2, 64, 12), (4, 4, 32, 1), (6, 2, 128, 24), (3, 1, 112, 2), (10, 2, 96, 16)])
def test_prefill_attention_whole_prompts(kernel_sets, Hq, Hkv, D, bs):
    """Whole prompts and long portions through the workgroup kernel: several sequences of
    uneven length, one of them continuing a cache of 100 tokens; page sizes that are powers of
    two (two neighbouring keys share a page), one, and no power of two; with and without a
    window (tiles that lie partly or wholly before the window's start)."""
    hip, _ = kernel_sets[torch.bfloat16]
    lens = [257, 33, 100 + 75, 16]
    slot, dense = make_paged_case(lens, Hq, Hkv, D, bs, torch.bfloat16, seed=D + 1)
    rows = [0] * 257 + [1] * 33 + [2] * 75 + [3] * 16
    pos = list(range(257)) + list(range(33)) + list(range(100, 175)) + list(range(16))
    q = rnd((len(rows), Hq, D), torch.bfloat16, 21)
    for window in (None, 40, 97):
        want = dense_attention(q, dense, rows, pos, D ** -0.5, window)
        for rt in (1, 2, 32, 64):        # 32: the 32 x 32 products (head sizes in steps of 32); 64: keys in two halves
            hip.attention_row_tiles = rt
            got = hip.paged_attention(q, slot, ctx_for(rows, pos), D ** -0.5, window)
            close(got.cpu(), want, torch.bfloat16)
    hip.attention_row_tiles = None


@pytest.mark.parametrize("start,T,row_tiles", [(1024, 1024, 64), (0, 1024, 64), (0, 1536, 32)])
def test_prefill_attention_long_portions_choose_the_32_row_products(kernel_sets, start, T, row_tiles):
    """Portions long enough that head size 128 goes to the 32-row products by itself
    (workgroups of 8 tokens x 16 heads of a group): 512 of them take the eight-wave form,
    each four waves on half of the keys, behind a context or from the start of a prompt; 768
    the four-wave form. One early key is made to stand out for one query."""
    hip, _ = kernel_sets[torch.bfloat16]
    Hq, Hkv, D, bs = 64, 4, 128, 16
    slot, dense = make_paged_case([start + T], Hq, Hkv, D, bs, torch.bfloat16, seed=5)
    rows, pos = [0] * T, list(range(start, start + T))
    q = rnd((T, Hq, D), torch.bfloat16, 22)
    k0, v0 = dense[0]
    q[700, 37] = (8.0 * k0[37 // 16, 3]).to(torch.bfloat16)         # query 700 of head 37 looks at key 3
    got = hip.paged_attention(q, slot, ctx_for(rows, pos), D ** -0.5)
    assert hip.last_attention_kernel == ("workgroup", row_tiles)
    want = dense_attention(q, dense, rows, pos, D ** -0.5)
    close(got.cpu(), want, torch.bfloat16)
    assert (got[700].view(Hq, D)[37].float().cpu() - v0[37 // 16, 3]).abs().max() < 0.05


@pytest.mark.parametrize("rise", [0.004, 0.05, -0.05])
def test_attention_scores_that_keep_rising(kernel_sets, rise):
    """Keys whose scores rise (or fall) steadily along the sequence: the running reference of
    the softmax has to follow, by small steps that stay under the threshold up to which the
    MFMA kernels leave it where it is (0.004: 7 bits over 600 keys; 0.05: 86 bits, a move every
    few tiles; -0.05: it stays at the first tile's), for a decoded token with and without key splits and for a prompt portion
    through every form of the workgroup kernel."""
    hip, _ = kernel_sets[torch.bfloat16]
    Hq, Hkv, D, bs, n = 8, 2, 64, 16, 600
    slot, dense = make_paged_case([n], Hq, Hkv, D, bs, torch.bfloat16, seed=3)
    g = torch.Generator().manual_seed(8)
    direction = torch.nn.functional.normalize(torch.randn(Hkv, D, generator=g), dim=-1)
    # key j of head h = noise + 8 rise j direction[h]; q = 2 direction[h] + noise: score 2 rise j, times log2 e in bits
    k_new = (0.1 * torch.randn(Hkv, n, D, generator=g) + rise * torch.arange(n)[None, :, None] * direction[:, None] * 8).to(torch.bfloat16)
    table = slot.block_table[0].tolist()
    for j in range(n):
        slot.k[table[j // bs], :, j % bs] = k_new[:, j].to(DEV)
    dense[0] = (k_new.float(), dense[0][1])
    q = (direction.repeat_interleave(Hq // Hkv, 0)[None] * 2 + 0.05 * torch.randn(40, Hq, D, generator=g)).to(torch.bfloat16).to(DEV)
    # a decoded token at the end
    want = dense_attention(q[:1], dense, [0], [n - 1], D ** -0.5)
    for splits in (None, (64, 10), (1 << 30, 1)):
        hip.attention_splits = splits
        close(hip.paged_attention(q[:1].contiguous(), slot, ctx_for([0], [n - 1]), D ** -0.5).cpu(), want, torch.bfloat16)
    hip.attention_splits = None
    # a portion of 40 tokens at the end
    rows, pos = [0] * 40, list(range(n - 40, n))
    want = dense_attention(q, dense, rows, pos, D ** -0.5)
    for rt in (1, 2, 32, 64):
        hip.attention_row_tiles = rt
        close(hip.paged_attention(q, slot, ctx_for(rows, pos), D ** -0.5).cpu(), want, torch.bfloat16)
    hip.attention_row_tiles = None


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("n,slot_idx", [(1, 0), (16, 15), (17, 16), (256, 255), (257, 256), (1024, 1023),
                                        (1, 1), (15, 15), (16, 16), (255, 255), (256, 256), (1024, 1024),
                                        (600, 127), (600, 128), (600, 255), (600, 256), (1100, 511),
                                        (1100, 512), (2048, 0), (2048, 1536)])
def test_attention_needles(kernel_sets, dtype, n, slot_idx):
    """The reference's needle vectors (tests/test_kernel_cuda.py:70-107): q = 0 makes every
    weight exactly 1/n; V is zero except one slot that holds 8 * (kv head + 1). The output is
    8 * (head // G + 1) / n if that slot is read and exactly 0 if it lies past the end."""
    hip, _ = kernel_sets[dtype]
    Hq, Hkv, D, bs = 32, 8, 128, 16
    nb = -(-max(n, slot_idx + 1) // bs)
    pages = torch.randperm(nb + 5)[:nb] + 1
    kp = torch.randn(nb + 6, Hkv, bs, D)
    vp = torch.zeros(nb + 6, Hkv, bs, D)
    for h in range(Hkv):
        vp[pages[slot_idx // bs], h, slot_idx % bs] = 8.0 * (h + 1)
    table = torch.zeros(1, 130, dtype=torch.int32)
    table[0, :nb] = pages.to(torch.int32)
    slot = SimpleNamespace(k=kp.to(dtype).to(DEV), v=vp.to(dtype).to(DEV), block_table=table.to(DEV),
                           block_size=bs, window=None)
    q = torch.zeros(1, Hq, D, dtype=dtype, device=DEV)
    G = Hq // Hkv
    head_val = torch.tensor([8.0 * (i // G + 1) for i in range(Hq)])
    want = (head_val / n if slot_idx < n else torch.zeros(Hq))[:, None].expand(Hq, D).reshape(1, Hq * D)
    for splits in (None, (128, 17), (256, 9), (512, 5)):
        hip.attention_splits = splits
        got = hip.paged_attention(q, slot, ctx_for([0], [n - 1]), 0.1)
        torch.testing.assert_close(got.float().cpu(), want, atol=1e-4, rtol=8e-3)
    hip.attention_splits = None


@pytest.mark.parametrize("dtype", DTYPES)
def test_attention_ignores_poison_past_the_end(kernel_sets, dtype):
    """inf / NaN in slots past each row's length, and in the null page, change nothing
    (tests/test_kernel_cuda.py:120-133)."""
    hip, _ = kernel_sets[dtype]
    lens = [20, 7, 300, 1025]
    slot, _ = make_paged_case(lens, 8, 2, 64, 16, dtype, seed=5)
    rows, pos = list(range(4)), [n - 1 for n in lens]
    q = rnd((4, 8, 64), dtype, 10)
    before = hip.paged_attention(q, slot, ctx_for(rows, pos), 0.125)
    for r, n in enumerate(lens):
        last = int(slot.block_table[r, (n - 1) // 16])
        if n % 16:
            slot.k[last, :, n % 16:] = float("inf")
            slot.v[last, :, n % 16:] = float("nan")
    slot.k[0] = float("nan")
    slot.v[0] = float("inf")
    after = hip.paged_attention(q, slot, ctx_for(rows, pos), 0.125)
    assert torch.isfinite(after).all()
    torch.testing.assert_close(after, before, atol=0, rtol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("Hq,Hkv,D,rot", [(4, 2, 16, 16), (8, 2, 32, 32), (6, 2, 48, 48), (3, 1, 128, 64),
                                          (2, 2, 256, 256)])
def test_qk_norm_rope_write(kernel_sets, dtype, Hq, Hkv, D, rot):
    from socrates_amd.cache import CacheManager
    from socrates_amd.parts import PagedKV
    hip, ref = kernel_sets[dtype]
    N, bs = 21, 8
    caches = [CacheManager([PagedKV(Hkv, D)], 3, 64, bs, 20, dtype, DEV) for _ in range(2)]
    rows, pos = [], []
    for c in caches:
        for n_tok in (9, 1, 11):
            r = c.open_row()
            if n_tok == 11:
                c.reserve(r, 30)
                c.advance(r, 19)                   # this row continues at position 19
            c.reserve(r, c.length(r) + n_tok)
        c.sync()
    for r, n_tok, start in ((0, 9, 0), (1, 1, 0), (2, 11, 19)):
        rows += [r] * n_tok
        pos += list(range(start, start + n_tok))
    positions = torch.tensor(pos, dtype=torch.int32, device=DEV)
    token_rows = torch.tensor(rows, dtype=torch.int32, device=DEV)
    qkv = rnd((N, (Hq + 2 * Hkv) * D), dtype, 12)
    qg, kg = (1 + 0.2 * torch.randn(D)).to(DEV), (1 + 0.2 * torch.randn(D)).to(DEV)
    inv_freq = (1.0 / (1e4 ** (torch.arange(0, rot, 2).float() / rot))).to(DEV)
    args = (qkv, Hq, Hkv, D, qg, kg, 1e-5, inv_freq, rot, positions, token_rows)
    got = hip.qk_norm_rope_write(*args, caches[0].slot(0))
    want = ref.qk_norm_rope_write(*args, caches[1].slot(0))
    close(got, want, dtype)
    close(caches[0].slot(0).k, caches[1].slot(0).k, dtype)
    close(caches[0].slot(0).v, caches[1].slot(0).v, dtype, atol=0, rtol=0)
    # the unfused pieces give the same
    q2, k2, v2 = hip.qk_norm_split(qkv, Hq, Hkv, D, qg, kg, 1e-5)
    hip.rope(q2, positions, inv_freq, rot)
    hip.rope(k2, positions, inv_freq, rot)
    close(q2, want, dtype)
    fresh = CacheManager([PagedKV(Hkv, D)], 3, 64, bs, 20, dtype, DEV)
    for n_tok in (9, 1, 30):
        fresh.reserve(fresh.open_row(), n_tok)
    fresh.sync()
    # same pages as caches[1]: both allocate 1, 2, 3, ... in the same order
    hip.kv_write(k2, v2, positions, token_rows, fresh.slot(0))
    close(fresh.slot(0).k, caches[1].slot(0).k, dtype)


@pytest.mark.parametrize("n0", [200, 900])
@pytest.mark.parametrize("Hq,Hkv,D,rope", [(32, 8, 128, True), (5, 1, 128, True), (6, 2, 64, True), (9, 3, 64, False),
                                           (4, 2, 128, False)])
def test_qk_norm_rope_write_long_prompts(kernel_sets, Hq, Hkv, D, rope, n0):
    """Hundreds of tokens in bfloat16 take the kernel that works on several heads per wave
    (head sizes 64 and 128, rotation over the whole head or none), from 1,024 tokens on its
    form with a token per wave (1,031 tokens: the last workgroup has three); head counts that
    do not fill the last wave, two rows, one of them continuing at position 37."""
    from socrates_amd.cache import CacheManager
    from socrates_amd.parts import PagedKV
    dtype = torch.bfloat16
    hip, ref = kernel_sets[dtype]
    bs = 16
    caches = [CacheManager([PagedKV(Hkv, D)], 2, 1024, bs, 80, dtype, DEV) for _ in range(2)]
    for c in caches:
        r0, r1 = c.open_row(), c.open_row()
        c.reserve(r0, n0)
        c.reserve(r1, 37)
        c.advance(r1, 37)
        c.reserve(r1, 37 + 131)
        c.sync()
    rows = [0] * n0 + [1] * 131
    pos = list(range(n0)) + list(range(37, 37 + 131))
    N = len(rows)
    positions = torch.tensor(pos, dtype=torch.int32, device=DEV)
    token_rows = torch.tensor(rows, dtype=torch.int32, device=DEV)
    qkv = rnd((N, (Hq + 2 * Hkv) * D), dtype, 31)
    qg, kg = (1 + 0.2 * torch.randn(D)).to(DEV), (1 + 0.2 * torch.randn(D)).to(DEV)
    inv_freq = (1.0 / (1e6 ** (torch.arange(0, D, 2).float() / D))).to(DEV) if rope else None
    args = (qkv, Hq, Hkv, D, qg, kg, 1e-6, inv_freq, D if rope else 0, positions, token_rows)
    got = hip.qk_norm_rope_write(*args, caches[0].slot(0))
    want = ref.qk_norm_rope_write(*args, caches[1].slot(0))
    close(got, want, dtype)
    close(caches[0].slot(0).k, caches[1].slot(0).k, dtype)
    close(caches[0].slot(0).v, caches[1].slot(0).v, dtype, atol=0, rtol=0)


def test_rope_properties(kernel_sets):
    """Position 0 is the identity; pair norms are kept; <rope(q, m), rope(k, n)> depends on
    m - n only; equals complex multiplication by e^{i pos theta^(-2j/D)}."""
    hip, _ = kernel_sets[torch.float32]
    D, theta = 32, 1e4
    inv_freq = (1.0 / (theta ** (torch.arange(0, D, 2).float() / D))).to(DEV)
    x = rnd((6, 1, D), torch.float32, 13)
    y = x.clone()
    hip.rope(y, torch.zeros(6, dtype=torch.int32, device=DEV), inv_freq, D)
    torch.testing.assert_close(y, x, atol=0, rtol=0)
    pos = torch.tensor([3, 10, 100, 1000, 4095, 7], dtype=torch.int32, device=DEV)
    y = x.clone()
    hip.rope(y, pos, inv_freq, D)
    z = torch.complex(x[..., :D // 2].double(), x[..., D // 2:].double()) * torch.polar(
        torch.ones(6, 1, D // 2, dtype=torch.float64, device=DEV),
        (pos.float()[:, None, None] * inv_freq).double())
    torch.testing.assert_close(y[..., :D // 2].double(), z.real, atol=1e-5, rtol=1e-5)
    torch.testing.assert_close(y[..., D // 2:].double(), z.imag, atol=1e-5, rtol=1e-5)
    q, k = rnd((1, 1, D), torch.float32, 14), rnd((1, 1, D), torch.float32, 15)
    dots = []
    for m, n in ((5, 2), (105, 102), (2003, 2000)):
        a, b = q.clone(), k.clone()
        hip.rope(a, torch.tensor([m], dtype=torch.int32, device=DEV), inv_freq, D)
        hip.rope(b, torch.tensor([n], dtype=torch.int32, device=DEV), inv_freq, D)
        dots.append((a * b).sum().item())
    # float32 angles resolve position * 2^-24 radians: the invariance holds to that
    bound = 4 * 2003 * 2.0 ** -24 * (q.norm() * k.norm()).item()
    assert max(dots) - min(dots) < bound
    assert abs(dots[0] - dots[1]) < 4 * 105 * 2.0 ** -24 * (q.norm() * k.norm()).item()


def test_sampling(kernel_sets):
    hip, ref = kernel_sets[torch.float32]
    V = 151936
    logits = rnd((5, V), torch.float32, 16, 3.0)
    logits[1, 777] = logits[1, 12345] = 50.0            # a tie: the lower index wins
    logits[2] = -1e30
    logits[2, V - 1] = 0.0
    assert hip.argmax(logits).tolist() == ref.argmax(logits).tolist()
    assert hip.argmax(logits)[1].item() == 777
    n = 64
    lg = rnd((n, 331), torch.float32, 17, 2.0)
    temp = torch.full((n,), 0.8, device=DEV)
    temp[::7] = 0.0
    seed = torch.arange(n, dtype=torch.int64, device=DEV) * 7919 + 1
    draws = torch.arange(n, dtype=torch.int64, device=DEV) % 5
    got = hip.sample(lg, temp, seed, draws).tolist()
    want = ref.sample(lg, temp, seed, draws).tolist()
    # the chosen token's CDF interval holds the uniform number (up to float32 rounding)
    agree = 0
    for i in range(n):
        if temp[i] == 0:
            assert got[i] == int(lg[i].argmax())
            continue
        p = torch.softmax(lg[i].double() / 0.8, -1).cpu()
        cdf = torch.cumsum(p, -1)
        u = uniform_of(int(seed[i]), int(draws[i]))
        lo = cdf[got[i] - 1].item() if got[i] else 0.0
        assert lo - 1e-5 <= u <= cdf[got[i]].item() + 1e-5
        agree += got[i] == want[i]
    assert agree >= n - 10 - 2
    # same (seed, draw) gives the same token whatever else is in the batch
    again = hip.sample(lg[10:20].contiguous(), temp[10:20].contiguous(), seed[10:20].contiguous(),
                       draws[10:20].contiguous()).tolist()
    assert again == got[10:20]
    # temperature to zero converges to argmax
    cold = hip.sample(lg, torch.full((n,), 1e-4, device=DEV), seed, draws)
    assert cold.tolist() == lg.argmax(-1).tolist()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("far", [0, 3, 15, 16, 17, 255, 256, 511])
def test_attention_far_key_stands_out(kernel_sets, dtype, far):
    """Among 700 near-uniform keys one far key matches the query strongly, so it takes almost
    all the weight: a kernel that skips it, or reads a neighbour instead (a page edge, a
    split seam), returns another value row by O(1), which random keys would hide."""
    hip, _ = kernel_sets[dtype]
    Hq, Hkv, D, bs, n = 8, 2, 64, 16, 700
    slot, dense = make_paged_case([n], Hq, Hkv, D, bs, dtype, seed=far + 1)
    u = torch.nn.functional.normalize(torch.randn(D), dim=0)
    q = (0.1 * torch.randn(1, Hq, D) + 6.0 * u).to(dtype).to(DEV)
    page, off = int(slot.block_table[0, far // bs]), far % bs
    slot.k[page, :, off] = (6.0 * u).to(dtype).to(DEV)
    slot.v[page, :, off] = torch.arange(D, dtype=torch.float32).to(dtype).to(DEV) / 8
    dense[0][0][:, far] = slot.k[page, :, off].float().cpu()
    dense[0][1][:, far] = slot.v[page, :, off].float().cpu()
    want = dense_attention(q, dense, [0], [n - 1], 1.0)
    assert (want.view(Hq, D) - slot.v[page, 0, off].float().cpu()).abs().max() < 0.05    # the far key dominates
    for splits in (None, (128, 6), (1 << 30, 1)):
        hip.attention_splits = splits
        got = hip.paged_attention(q, slot, ctx_for([0], [n - 1]), 1.0)
        close(got.cpu(), want, dtype, atol=3e-5 if dtype == torch.float32 else 3e-2)
    hip.attention_splits = None


@pytest.mark.parametrize("Hq,Hkv,n", [(8, 2, 20000), (16, 4, 16448), (4, 1, 33000)])
def test_decoded_token_behind_a_long_context(kernel_sets, Hq, Hkv, n):
    """One decoded token behind tens of thousands of keys, at head counts for which the planner
    once asked for more key splits than the merge kernel holds (313, 257 and 512): the plan
    stays within the limit and the result equals plain attention, with one far key made to
    stand out so that a split that is skipped or merged wrongly shows."""
    from socrates_amd.kernels import MAX_KEY_SPLITS, KernelError
    hip, _ = kernel_sets[torch.bfloat16]
    D, bs = 64, 16
    slot, dense = make_paged_case([n], Hq, Hkv, D, bs, torch.bfloat16, seed=n)
    far = n // 3 + 5
    u = torch.nn.functional.normalize(torch.randn(D), dim=0)
    q = (0.1 * torch.randn(1, Hq, D) + 4.0 * u).to(torch.bfloat16).to(DEV)
    page, off = int(slot.block_table[0, far // bs]), far % bs
    slot.k[page, :, off] = (4.0 * u).to(torch.bfloat16).to(DEV)
    dense[0][0][:, far] = slot.k[page, :, off].float().cpu()
    split_len, n_splits = hip.plan_mfma(1, Hkv, Hq // Hkv, n)
    assert n_splits <= MAX_KEY_SPLITS and n_splits * split_len >= n
    want = dense_attention(q, dense, [0], [n - 1], 1.0)
    got = hip.paged_attention(q, slot, ctx_for([0], [n - 1]), 1.0)
    assert hip.last_attention_kernel[0] == "wave"
    close(got.cpu(), want, torch.bfloat16, atol=3e-2)
    # an override beyond the limit is refused on the host, with the limit in the message
    hip.attention_splits = (16, 100000)
    try:
        with pytest.raises(KernelError, match="at most 256"):
            hip.paged_attention(q, slot, ctx_for([0], [n - 1]), 1.0)
    finally:
        hip.attention_splits = None
