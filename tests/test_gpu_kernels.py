"""Each kernel alone against a plain PyTorch float32/float64 reference of the same
op, at sizes other than the engine's tiny models (odd widths, other head sizes
and group sizes, larger pages, fragmented block tables).  Where random inputs
would hide a fault, one score is made to stand out."""

import math

import pytest
import torch

from tests.plain import qwen2_plain as plain

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def K():
    from paged_attention_engine_amd.kernels import lib
    return lib


def tol(dtype, scale=1.0):
    return (2e-6 if dtype == "float32" else 2.0 ** -7) * scale


# ------------------------------------------------------------------ small row-wise kernels
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding(dtype):
    table = torch.randn(301, 72).to(DT[dtype])
    ids = torch.tensor([5, 300, 0, 5, 17], dtype=torch.int32)
    out = torch.empty(5, 72, dtype=torch.float32, device=DEV)
    K().embedding(out, table.to(DEV), ids.to(DEV))
    assert torch.equal(out.cpu(), table[ids.long()].float())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [72, 1536, 1000])
def test_add_rmsnorm(dtype, hidden):
    torch.manual_seed(0)
    n, eps = 7, 1e-5
    res = torch.randn(n, hidden) * 3
    delta = torch.randn(n, hidden).to(DT[dtype])
    w = (1 + 0.1 * torch.randn(hidden)).to(DT[dtype])
    summed = res + delta.float()
    # reference: normalise in float32, round to the storage type, multiply by the weight, round
    normed = (summed * torch.rsqrt(summed.pow(2).mean(-1, keepdim=True) + eps)).to(DT[dtype])
    want = (w.float() * normed.float()).to(DT[dtype]).float()
    r = res.to(DEV)
    out = torch.empty(n, hidden, dtype=DT[dtype], device=DEV)
    K().add_rmsnorm(r, delta.to(DEV), w.to(DEV), eps, out)
    assert torch.allclose(r.cpu(), summed, atol=1e-6)  # the sum is formed and kept in float32
    assert (out.float().cpu() - want).abs().max() <= tol(dtype, float(want.abs().max()))
    # gather of selected rows: nothing is written back; a float32 weight is taken as stored
    rows = torch.tensor([6, 0, 3], dtype=torch.int32, device=DEV)
    r2 = res.to(DEV)
    out2 = torch.empty(3, hidden, dtype=DT[dtype], device=DEV)
    K().add_rmsnorm(r2, delta.to(DEV), w.float().to(DEV), eps, out2, rows)
    assert torch.equal(r2.cpu(), res)
    assert (out2.float().cpu() - want[[6, 0, 3]]).abs().max() <= tol(dtype, float(want.abs().max()))
    # no pending branch: plain norm of the residual; zero rows give zero, not NaN
    r3 = torch.zeros(2, hidden, device=DEV)
    out3 = torch.empty(2, hidden, dtype=DT[dtype], device=DEV)
    K().add_rmsnorm(r3, None, w.to(DEV), eps, out3)
    assert torch.equal(out3.float().cpu(), torch.zeros(2, hidden))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("M,N,K_", [(1, 50, 72), (70, 193, 100), (5, 1000, 353), (64, 64, 16)])
def test_gemm_plain(dtype, M, N, K_):
    torch.manual_seed(1)
    a = torch.randn(M, K_).to(DT[dtype])
    w = torch.randn(N, K_).to(DT[dtype])
    b = torch.randn(N).to(DT[dtype])
    want = a.double() @ w.double().t() + b.double()
    out = torch.empty(M, N, dtype=DT[dtype], device=DEV)
    K().gemm_plain(out, a.to(DEV), w.to(DEV), b.to(DEV))
    assert (out.double().cpu() - want).abs().max() <= tol(dtype, float(want.abs().max())) * (4 if dtype == "float32" else 1)
    if dtype == "bfloat16":  # float32 results from bfloat16 operands (the head's product)
        out32 = torch.empty(M, N, dtype=torch.float32, device=DEV)
        K().gemm_plain(out32, a.to(DEV), w.to(DEV), None)
        assert (out32.double().cpu() - (want - b.double())).abs().max() <= 1e-5 * float(want.abs().max())
    else:  # a row's result does not depend on the rows beside it
        one = torch.empty(1, N, dtype=torch.float32, device=DEV)
        K().gemm_plain(one, a[M - 1:].to(DEV), w.to(DEV), b.to(DEV))
        assert torch.equal(one[0], out[M - 1])


@pytest.mark.parametrize("M", [1, 8, 17, 64])
@pytest.mark.parametrize("N,K_", [(2048, 1536), (1536, 8960), (50, 72), (777, 64), (96, 200),
                                  # about 256 workgroups of 5, 6, 7 and 8 wavefronts of 16 weight rows (above 16 rows of A)
                                  (17930, 72), (22000, 136), (27640, 72), (32000, 40),
                                  # over a thousand workgroups of 32 weight rows: those already at 8 rows of A
                                  (33000, 40)])
def test_gemm_skinny(M, N, K_):
    torch.manual_seed(M + N)
    a = (torch.randn(M, K_) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, K_) * 0.1).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16)
    want = a.double() @ w.double().t()
    scale = float(want.abs().max())
    # bfloat16 out with bias
    out = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
    K().gemm_skinny(out, a.to(DEV), w.to(DEV), b.to(DEV), K().EPI_BF16)
    assert (out.double().cpu() - (want + b.double())).abs().max() <= 2.0 ** -7 * (scale + 3)
    # float32 out: one range, and partial sums over several k ranges added in order
    out32 = torch.empty(M, N, dtype=torch.float32, device=DEV)
    K().gemm_skinny(out32, a.to(DEV), w.to(DEV), None, K().EPI_F32)
    assert (out32.double().cpu() - want).abs().max() <= 2e-5 * scale
    for splits in {K().skinny_splits(N, K_, M), 3 if K_ >= 1536 else 1}:  # the rule's choice, and three ranges
        parts = torch.full((splits, M, N), float("nan"), dtype=torch.float32, device=DEV)
        K().gemm_skinny(parts, a.to(DEV), w.to(DEV), None, K().EPI_F32, splits)
        assert (parts.sum(0).double().cpu() - want).abs().max() <= 2e-5 * scale
    # a row's result does not depend on the other rows (up to 16 rows always; above, where the many
    # weight rows of the last four shapes do not bring in a kernel that adds k in another order)
    if M > 1 and (M <= 16 or N < 4096):
        one = torch.empty(1, N, dtype=torch.float32, device=DEV)
        K().gemm_skinny(one, a[M - 1:].to(DEV), w.to(DEV), None, K().EPI_F32)
        assert torch.equal(one[0], out32[M - 1])


@pytest.mark.parametrize("M", [1, 8, 12, 17, 40, 64])
@pytest.mark.parametrize("N,K_,ranges", [(1536, 1536, 4), (1536, 8960, 5), (200, 72, 1), (72, 200, 1), (3584, 512, 2),
                                          (8192, 1024, 3),
                                          # more shares a row than a workgroup's threads read in one trip (512 with up
                                          # to 16 rows, 256 above), in whole groups of four and not
                                          (8256, 64, 1), (8264, 72, 1)])
def test_a_norm_folded_into_the_products_around_it(M, N, K_, ranges):
    """The product that ends a branch adds itself into the float32 residual and leaves, for the
    product after the next norm, the rows bfloat16(residual * w_norm) and the shares of every
    row's sum of squares; that product multiplies its sums by rsqrt(mean square + eps).  Together
    they give what add + RMSNorm + product give, without a norm kernel in between."""
    torch.manual_seed(M * 7 + N)
    eps = 1e-5
    a = (torch.randn(M, K_) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, K_) * 0.1).to(torch.bfloat16)
    residual = torch.randn(M, N) * 2.0
    w_norm = (1 + 0.2 * torch.randn(N)).to(torch.bfloat16)
    want_residual = residual.double() + a.double() @ w.double().t()
    res_d = residual.to(DEV)
    next_rows = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    stats = torch.full((M, K().stat_tiles(N)), float("nan"), dtype=torch.float32, device=DEV)
    K().gemm_skinny(res_d, a.to(DEV), w.to(DEV), None, K().EPI_RESIDUAL, ranges,
                    following=(next_rows, w_norm.to(DEV), stats))
    top = float(want_residual.abs().max())
    assert (res_d.double().cpu() - want_residual).abs().max() <= 2e-5 * top
    want_rows = (res_d.cpu() * w_norm.float()).to(torch.bfloat16)
    assert (next_rows.float().cpu() - want_rows.float()).abs().max() <= 2.0 ** -7 * float(want_rows.float().abs().max())
    assert torch.allclose(stats.sum(1).double().cpu(), res_d.double().cpu().pow(2).sum(1), rtol=1e-5)
    # the same again lands on top of the first (the residual is updated in place)
    K().gemm_skinny(res_d, a.to(DEV), w.to(DEV), None, K().EPI_RESIDUAL, 1, following=(next_rows, w_norm.to(DEV), stats))
    want2 = want_residual + a.double() @ w.double().t()
    assert (res_d.double().cpu() - want2).abs().max() <= 4e-5 * float(want2.abs().max())

    # the consumer: a product over the rows whose scale is owed, against norm-then-product
    x = res_d.double().cpu()
    normed = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w_norm.double()
    if N % 8:
        return  # the consumer's inner size must be a multiple of 8
    for N2 in (48, 1000):
        w2 = (torch.randn(N2, N) * 0.1).to(torch.bfloat16)
        b2 = torch.randn(N2).to(torch.bfloat16)
        want = normed @ w2.double().t() + b2.double()
        out = torch.empty(M, N2, dtype=torch.bfloat16, device=DEV)
        K().gemm_skinny(out, next_rows, w2.to(DEV), b2.to(DEV), K().EPI_BF16, row_scale=(stats, eps))
        assert (out.double().cpu() - want).abs().max() <= 2.0 ** -6 * (float(want.abs().max()) + 1)
        splits = 2 if N >= 1024 else 1
        out2 = torch.empty(M, N2, dtype=torch.bfloat16, device=DEV)
        K().gemm_skinny(out2, next_rows, w2.to(DEV), b2.to(DEV), K().EPI_BF16, splits, row_scale=(stats, eps))
        assert (out2.double().cpu() - want).abs().max() <= 2.0 ** -6 * (float(want.abs().max()) + 1)
    # rows whose scale is paid by a kernel of its own, for parts that want plain activations
    plain_rows = K().scaled_rows(next_rows, stats, eps)
    assert (plain_rows.double().cpu() - normed).abs().max() <= 2.0 ** -6 * float(normed.abs().max())


@pytest.mark.parametrize("N,K_", [(1536, 1536), (1536, 8960), (2048, 1536), (17920, 1536), (3584, 18944), (4608, 3584),
                                  (200, 1032), (1000, 264)])
def test_a_rows_sums_do_not_depend_on_the_batch_up_to_16_rows(N, K_):
    """Up to 16 rows every product takes its k ranges from its sizes alone and adds them in one order,
    whichever kernel runs them (one workgroup of sixteen wavefronts for four ranges side by side, or
    a workgroup per range and a ticket): a row alone, among 8 rows and among 16 gives the same bits,
    through the plain, the gated and the residual epilogue, with and without a row scale."""
    torch.manual_seed(N + K_)
    a = (torch.randn(16, K_) * 0.5).to(torch.bfloat16).to(DEV)
    w = (torch.randn(N, K_) * 0.1).to(torch.bfloat16).to(DEV)
    stats_in = (torch.rand(16, K().stat_tiles(K_)) + 0.5).to(DEV)
    residual = (torch.randn(16, N) * 2.0).to(DEV)
    w_norm = (1 + 0.2 * torch.randn(N)).to(torch.bfloat16).to(DEV)

    def run(rows, epilogue, scaled):
        M = len(rows)
        x = a[rows].contiguous()
        scale = (stats_in[rows].contiguous(), 1e-6) if scaled else None
        if epilogue == K().EPI_RESIDUAL:
            out = residual[rows].clone()
            nxt = torch.empty(M, N, dtype=torch.bfloat16, device=DEV)
            stats = torch.empty(M, K().stat_tiles(N), dtype=torch.float32, device=DEV)
            K().gemm_skinny(out, x, w, None, epilogue, K().residual_splits(N, K_, M), scale, (nxt, w_norm, stats))
            return out, nxt, stats
        cols = N // 2 if epilogue == K().EPI_SWIGLU else N
        out = torch.empty(M, cols, dtype=torch.bfloat16, device=DEV)
        K().gemm_skinny(out, x, w, None, epilogue, K().whole_sum_splits(N, K_, M), scale)
        return (out,)

    epilogues = [K().EPI_BF16, K().EPI_RESIDUAL] + ([K().EPI_SWIGLU] if N % 16 == 0 else [])
    for epilogue in epilogues:
        for scaled in (False, True):
            alone = run([5], epilogue, scaled)
            eight = run(list(range(8)), epilogue, scaled)
            twelve = run(list(range(2, 14)), epilogue, scaled)
            sixteen = run(list(range(16)), epilogue, scaled)
            for t_alone, t8, t12, t16 in zip(alone, eight, twelve, sixteen):
                assert torch.equal(t_alone[0], t8[5]) and torch.equal(t_alone[0], t12[3]) and torch.equal(t_alone[0], t16[5])
    # four ranges side by side in one workgroup are the four ranges of separate workgroups, bit for bit
    # (where a decode program has the LDS for one range's activations)
    if K().residual_splits(N, K_, 8) == 4 and K().program_takes_product(8, K_, 4, quad_bytes=6144):
        side_by_side = run(list(range(8)), K().EPI_RESIDUAL, True)
        program = K().DecodeProgram(DEV, 2)  # a decode program's product phase always goes by tickets
        out = residual[:8].clone()
        nxt = torch.empty(8, N, dtype=torch.bfloat16, device=DEV)
        stats = torch.empty(8, K().stat_tiles(N), dtype=torch.float32, device=DEV)
        with K().recording(program):
            K().gemm_skinny(out, a[:8].contiguous(), w, None, K().EPI_RESIDUAL, 4, (stats_in[:8].contiguous(), 1e-6),
                            (nxt, w_norm, stats))
        program.launch()
        torch.cuda.synchronize()
        program.check()
        for got, want in zip((out, nxt, stats), side_by_side):
            assert torch.equal(got, want)


@pytest.mark.parametrize("M,N,K_,ranges", [(8, 1536, 8960, 1), (8, 1536, 1536, 4), (12, 18944, 3584, 1), (16, 3584, 18944, 4),
                                            (7, 1000, 1032, 3), (16, 72, 2048, 4), (3, 200, 8, 1)])
def test_the_residual_epilogue_on_every_branch_of_its_launcher(M, N, K_, ranges):
    """One range, four ranges side by side in a workgroup of sixteen wavefronts, ticketed ranges, a
    width that is no multiple of 16: the residual, the next rows and the sums of squares against a
    float64 computation, tightly."""
    torch.manual_seed(M + N + K_)
    a = (torch.randn(M, K_) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, K_) * 0.1).to(torch.bfloat16)
    residual = torch.randn(M, N) * 2.0
    w_norm = (1 + 0.2 * torch.randn(N)).to(torch.bfloat16)
    want = residual.double() + a.double() @ w.double().t()
    res_d = residual.to(DEV)
    nxt = torch.full((M, N), float("nan"), dtype=torch.bfloat16, device=DEV)
    stats = torch.full((M, K().stat_tiles(N)), float("nan"), dtype=torch.float32, device=DEV)
    K().gemm_skinny(res_d, a.to(DEV), w.to(DEV), None, K().EPI_RESIDUAL, ranges, following=(nxt, w_norm.to(DEV), stats))
    top = float(want.abs().max())
    assert (res_d.double().cpu() - want).abs().max() <= 4e-6 * top + 1e-6
    rows = (res_d.cpu() * w_norm.float()).to(torch.bfloat16)
    assert torch.equal(nxt.cpu(), rows)  # the rounding of exactly the residual that was written
    assert torch.isfinite(stats).all()
    assert torch.allclose(stats.double().cpu().sum(1), res_d.double().cpu().pow(2).sum(1), rtol=2e-6)
    # every share is its own 16 columns' sum of squares
    padded = torch.zeros(M, K().stat_tiles(N) * 16, dtype=torch.float64)
    padded[:, :N] = res_d.double().cpu().pow(2)
    assert torch.allclose(stats.double().cpu(), padded.view(M, -1, 16).sum(-1), rtol=2e-6, atol=1e-12)
    K().check_tickets_zero(DEV)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_rows(dtype):
    torch.manual_seed(3)
    V, H, T = 333, 200, 9
    table = torch.randn(V, H).to(DT[dtype])
    ids = torch.randint(0, V, (T,), dtype=torch.int32)
    w_norm = (1 + 0.1 * torch.randn(H)).to(torch.bfloat16)
    residual = torch.empty(T, H, dtype=torch.float32, device=DEV)
    rows = torch.empty(T, H, dtype=torch.bfloat16, device=DEV)
    stats = torch.empty(T, K().stat_tiles(H), dtype=torch.float32, device=DEV)
    K().embedding_rows(residual, table.to(DEV), ids.to(DEV), 1.5, rows, w_norm.to(DEV), stats)
    want = 1.5 * table[ids.long()].float()
    assert torch.equal(residual.cpu(), want)
    assert torch.equal(rows.cpu(), (want * w_norm.float()).to(torch.bfloat16))
    assert torch.allclose(stats.sum(1).cpu(), want.pow(2).sum(1), rtol=1e-5)
    assert torch.allclose(stats[:, -1].cpu(), want[:, 192:].pow(2).sum(1), rtol=1e-5)  # the last, short tile


@pytest.mark.parametrize("M", [9, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K_", [(32777, 264), (9000, 1024), (151936, 72)])
def test_gemm_many_weight_rows(M, N, K_):
    """More than 16 rows of activations and many weight rows take the kernel that shares the
    activations through LDS (a width and a depth that are no multiples of its tiles among them)."""
    torch.manual_seed(M + N)
    a = (torch.randn(M, K_) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, K_) * 0.1).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16)
    want = a.double() @ w.double().t()
    scale = float(want.abs().max())
    d_a, d_w = a.to(DEV), w.to(DEV)
    out = torch.full((M, N), 77.0, dtype=torch.bfloat16, device=DEV)
    K().gemm_skinny(out, d_a, d_w, b.to(DEV), K().EPI_BF16)
    assert (out.double().cpu() - (want + b.double())).abs().max() <= 2.0 ** -7 * (scale + 3)
    out32 = torch.full((M, N), 77.0, dtype=torch.float32, device=DEV)
    K().gemm_skinny(out32, d_a, d_w, None, K().EPI_F32)
    assert (out32.double().cpu() - want).abs().max() <= 2e-5 * scale
    splits = 4 if K_ >= 1024 else 1  # 71 groups of 128 weight rows x 4 k ranges: still this kernel
    parts = torch.full((splits, M, N), float("nan"), dtype=torch.float32, device=DEV)
    K().gemm_skinny(parts, d_a, d_w, None, K().EPI_F32, splits)
    assert (parts.sum(0).double().cpu() - want).abs().max() <= 2e-5 * scale
    if K_ > 128:  # the bias epilogue over several k ranges: partial sums are added up inside the kernel
        ranges = 4 if K_ >= 1024 else 2
        for _ in range(2):  # the second call finds the tickets as the first left them
            out_k = torch.full((M, N), 77.0, dtype=torch.bfloat16, device=DEV)
            K().gemm_skinny(out_k, d_a, d_w, b.to(DEV), K().EPI_BF16, ranges)
            assert int(K().skinny_tickets(DEV).abs().sum()) == 0
            assert (out_k.double().cpu() - (want + b.double())).abs().max() <= 2.0 ** -7 * (scale + 3)
    # a row alone goes through the few-row kernel, which adds in another order: equal to rounding
    one = torch.empty(1, N, dtype=torch.float32, device=DEV)
    K().gemm_skinny(one, d_a[M - 1:], d_w, None, K().EPI_F32)
    assert (one[0] - out32[M - 1]).abs().max() <= 2e-5 * scale


def test_sums_over_k_ranges_inside_the_kernel_are_repeatable():
    """Partial sums are added in range order whichever workgroup comes last, so a product gives the
    same bits every time; two inputs take turns, so that a partial sum left over from the launch
    before (or read before it was written) would show."""
    torch.manual_seed(11)
    M, inter, K_, ranges = 64, 18944, 1024, 3
    w = (torch.randn(2 * inter, K_) * 0.05).to(torch.bfloat16).to(DEV)
    inputs = [torch.randn(M, K_).to(torch.bfloat16).to(DEV) for _ in range(2)]
    first = []
    for a in inputs:
        out = torch.empty(M, inter, dtype=torch.bfloat16, device=DEV)
        K().gemm_skinny(out, a, w, None, K().EPI_SWIGLU, ranges)
        first.append(out)
    one_range = torch.empty(M, inter, dtype=torch.bfloat16, device=DEV)
    K().gemm_skinny(one_range, inputs[0], w, None, K().EPI_SWIGLU)
    assert (one_range.float() - first[0].float()).abs().max() <= 2.0 ** -6 * float(one_range.float().abs().max())
    different = 0
    for i in range(400):
        out = torch.empty(M, inter, dtype=torch.bfloat16, device=DEV)
        K().gemm_skinny(out, inputs[i % 2], w, None, K().EPI_SWIGLU, ranges)
        different += int(not torch.equal(out, first[i % 2]))
    assert different == 0
    assert int(K().skinny_tickets(DEV).abs().sum()) == 0


@pytest.mark.parametrize("M", [17, 48, 64])
def test_gemm_partial_sums_on_small_workgroups(M):
    """Weight rows too few for 128-row workgroups to fill the chip, enough k ranges for 64-row ones:
    the float32 partial sums come from the many-weight-rows kernel's smaller workgroups."""
    torch.manual_seed(M)
    N, K_, ranges = 3584, 2048, 8
    a = (torch.randn(M, K_) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, K_) * 0.1).to(torch.bfloat16)
    want = a.double() @ w.double().t()
    parts = torch.full((ranges, M, N), float("nan"), dtype=torch.float32, device=DEV)
    K().gemm_skinny(parts, a.to(DEV), w.to(DEV), None, K().EPI_F32, ranges)
    assert (parts.sum(0).double().cpu() - want).abs().max() <= 2e-5 * float(want.abs().max())
    # each range holds its own part of the sum
    k_per = K_ // ranges
    first = a[:, :k_per].double() @ w[:, :k_per].double().t()
    assert (parts[0].double().cpu() - first).abs().max() <= 2e-5 * float(want.abs().max())


@pytest.mark.parametrize("M", [1, 8, 13, 33, 64])
@pytest.mark.parametrize("inter,K_", [(8960, 1536), (176, 64), (48, 72), (40, 72), (37888, 136),
                                      (11008, 264), (13824, 136), (16000, 72)])  # workgroups of 6, 7, 8 wavefronts
def test_gemm_skinny_gated(M, inter, K_):
    torch.manual_seed(inter)
    a = torch.randn(M, K_).to(torch.bfloat16)
    gate = (torch.randn(inter, K_) * 0.2).to(torch.bfloat16)
    up = (torch.randn(inter, K_) * 0.2).to(torch.bfloat16)
    want = plain.silu(a.double() @ gate.double().t()) * (a.double() @ up.double().t())
    w = torch.stack([gate.view(inter // 8, 8, K_), up.view(inter // 8, 8, K_)], dim=1).reshape(2 * inter, K_)
    out = torch.empty(M, inter, dtype=torch.bfloat16, device=DEV)
    K().gemm_skinny(out, a.to(DEV), w.contiguous().to(DEV), None, K().EPI_SWIGLU)
    assert (out.double().cpu() - want).abs().max() <= 2.0 ** -7 * float(want.abs().max())
    # several k ranges, added up inside the kernel (twice: the tickets are back at zero in between)
    if K_ > 128:
        for _ in range(2):
            out_k = torch.full_like(out, 3.0)
            K().gemm_skinny(out_k, a.to(DEV), w.contiguous().to(DEV), None, K().EPI_SWIGLU, min(3, -(-K_ // 128)))
            assert int(K().skinny_tickets(DEV).abs().sum()) == 0
            assert (out_k.double().cpu() - want).abs().max() <= 2.0 ** -7 * float(want.abs().max())
    # the separate gate kernel reads the same interleaved layout
    both = (a.double() @ w.double().t()).to(torch.bfloat16)
    out2 = torch.empty(M, inter, dtype=torch.bfloat16, device=DEV)
    K().swiglu(out2, both.to(DEV), 8)
    assert (out2.double().cpu() - want).abs().max() <= 2.0 ** -6 * float(want.abs().max())


def test_add_rmsnorm_sums_float32_partials_in_order():
    torch.manual_seed(4)
    n, hidden, eps = 5, 200, 1e-6
    res = torch.randn(n, hidden)
    parts = torch.randn(3, n, hidden)
    w = (1 + 0.1 * torch.randn(hidden)).to(torch.bfloat16)
    summed = res + ((parts[0] + parts[1]) + parts[2])
    normed = (summed * torch.rsqrt(summed.pow(2).mean(-1, keepdim=True) + eps)).to(torch.bfloat16)
    want = (w.float() * normed.float()).to(torch.bfloat16).float()
    r = res.to(DEV)
    out = torch.empty(n, hidden, dtype=torch.bfloat16, device=DEV)
    K().add_rmsnorm(r, parts.to(DEV), w.to(DEV), eps, out)
    assert torch.allclose(r.cpu(), summed, atol=1e-6)
    assert (out.float().cpu() - want).abs().max() <= 2.0 ** -7 * float(want.abs().max())
    rows = torch.tensor([4, 1], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, hidden, dtype=torch.bfloat16, device=DEV)
    K().add_rmsnorm(res.to(DEV), parts.to(DEV), w.to(DEV), eps, out2, rows)
    assert (out2.float().cpu() - want[[4, 1]]).abs().max() <= 2.0 ** -7 * float(want.abs().max())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_swiglu(dtype):
    x = (torch.randn(9, 2 * 177) * 3).to(DT[dtype])
    x[0, :5] = torch.tensor([0.0, -30.0, 30.0, -100.0, 100.0]).to(DT[dtype])
    want = plain.silu(x[:, :177].double()) * x[:, 177:].double()
    out = torch.empty(9, 177, dtype=DT[dtype], device=DEV)
    K().swiglu(out, x.to(DEV))
    assert torch.isfinite(out).all()
    assert (out.double().cpu() - want).abs().max() <= tol(dtype, float(want.abs().max()))


# ------------------------------------------------------------------ paged cache helpers
def scattered_tables(seq_lens, bs, num_blocks, seed=0, width=None):
    """Block tables drawn from a shuffled pool: descending, non-adjacent, fragmented
    (the reference fragments its pool for the same reason, tests/test_parity.py:196-223)."""
    gen = torch.Generator().manual_seed(seed)
    order = torch.randperm(num_blocks, generator=gen).tolist()
    need = [-(-n // bs) for n in seq_lens]
    assert sum(need) <= num_blocks
    width = width or max(need)
    tables = torch.full((len(seq_lens), width), -1, dtype=torch.int32)
    for s, n in enumerate(need):
        tables[s, :n] = torch.tensor([order.pop() for _ in range(n)], dtype=torch.int32)
    return tables


def fill_pools(keys, values, tables, bs, num_blocks, dtype):
    """keys/values: per sequence [n, nkv, hd].  Pools: K [nb][nkv][bs][hd], V [nb][nkv][hd][bs]."""
    nkv, hd = keys[0].shape[1:]
    kp = torch.zeros(num_blocks, nkv, bs, hd, dtype=dtype)
    vp = torch.zeros(num_blocks, nkv, hd, bs, dtype=dtype)
    for s, (k, v) in enumerate(zip(keys, values)):
        for p in range(k.shape[0]):
            blk = int(tables[s, p // bs])
            if blk < 0:
                continue  # a page the window has passed: given back, nothing of it is in the pool
            kp[blk, :, p % bs, :] = k[p].to(dtype)
            vp[blk, :, :, p % bs] = v[p].to(dtype)
    return kp, vp


def reference_attention(q, k, v, pos, scale, window):
    """One query (nh, hd) at position `pos` over keys/values [n, nkv, hd] in float64."""
    nh, nkv = q.shape[0], k.shape[1]
    g = nh // nkv
    start = max(0, pos - window + 1) if window else 0
    out = torch.empty(nh, v.shape[-1], dtype=torch.float64)
    for h in range(nh):
        kk = k[start:pos + 1, h // g].double()
        vv = v[start:pos + 1, h // g].double()
        w = torch.softmax((kk @ q[h].double()) * scale, 0)
        out[h] = w @ vv
    return out


# ------------------------------------------------------------------ rotation and cache write
def test_rope_table():
    """Angles are position * inv_freq in float32 (engine/model.py:138-152 of the reference)."""
    positions = torch.tensor([0, 1, 2, 77, 4095, 32767, 131071], dtype=torch.int32)
    inv = plain.rope_inv_freq(48, 1e6)
    got = K().rope_table(positions.to(DEV), inv.to(DEV)).cpu()
    angle = (positions.float()[:, None] * inv[None, :]).double()  # the float32 product, as the reference forms it
    assert got.shape == (7, 24, 2)
    assert (got[..., 0].double() - angle.cos()).abs().max() <= 2e-6
    assert (got[..., 1].double() - angle.sin()).abs().max() <= 2e-6


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,rot,bs", [(4, 2, 16, 16, 4), (6, 1, 48, 48, 16), (3, 3, 32, 16, 8),
                                              (12, 2, 128, 128, 16), (5, 1, 24, 8, 4), (2, 1, 20, 12, 4)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_rope_kv_write(dtype, nh, nkv, hd, rot, bs, with_bias):
    """`with_bias`: the rows come without the projection's bias, which the kernel adds first (rounded
    to the storage type, as the projection's own epilogue would) before it rotates and stores."""
    torch.manual_seed(2)
    theta = 50000.0
    # two sequences: one brings positions 5..11, the other the single position 37
    positions = list(range(5, 12)) + [37]
    tok_seq = [0] * 7 + [1]
    tables = scattered_tables([12, 38], bs, 40, seed=3)
    T = len(positions)
    qkv = torch.randn(T, (nh + 2 * nkv) * hd).to(DT[dtype])
    pos_d = torch.tensor(positions, dtype=torch.int32, device=DEV)
    table = K().rope_table(pos_d, plain.rope_inv_freq(rot, theta).to(DEV))
    kp = torch.full((40, nkv, bs, hd), 7.0, dtype=DT[dtype])
    vp = torch.full((40, nkv, hd, bs), 7.0, dtype=DT[dtype])
    d_qkv, d_kp, d_vp = qkv.to(DEV), kp.to(DEV), vp.to(DEV)
    bias = torch.randn((nh + 2 * nkv) * hd).to(DT[dtype]) if with_bias else None
    K().rope_kv_write(d_qkv, nh, nkv, hd, rot, table, pos_d,
                      torch.tensor(tok_seq, dtype=torch.int32, device=DEV), tables.to(DEV), bs, d_kp, d_vp,
                      bias.to(DEV) if with_bias else None)
    if with_bias:
        qkv = (qkv.float() + bias.float()).to(DT[dtype])
    x = qkv.double().view(T, nh + 2 * nkv, hd)
    cos, sin = plain.rope_cos_sin(plain.rope_inv_freq(rot, theta, torch.float64), torch.tensor(positions), torch.float64)
    rotated = x.clone()
    rotated[..., :rot] = x[..., :rot] * cos[:, None] + plain.rotate_half(x[..., :rot]) * sin[:, None]
    got_q = d_qkv.cpu().double().view(T, nh + 2 * nkv, hd)[:, :nh]
    bound = tol(dtype, 4.0) if dtype == "bfloat16" else 2e-5  # float32 angles up to 37 rad
    assert (got_q - rotated[:, :nh]).abs().max() <= bound
    # keys (rotated) and values (raw) sit at block_table[pos // bs] * bs + pos % bs; nothing else changed
    want_k, want_v = kp.clone().double(), vp.clone().double()
    for t, (p, s) in enumerate(zip(positions, tok_seq)):
        blk = int(tables[s, p // bs])
        want_k[blk, :, p % bs, :] = rotated[t, nh:nh + nkv]
        want_v[blk, :, :, p % bs] = x[t, nh + nkv:]
    assert (d_kp.cpu().double() - want_k).abs().max() <= bound
    assert torch.equal(d_vp.cpu().double(), want_v)
    untouched = torch.ones(40, dtype=torch.bool)
    for p, s in zip(positions, tok_seq):
        untouched[int(tables[s, p // bs])] = False
    assert torch.equal(d_kp.cpu()[untouched], kp[untouched])


@pytest.mark.parametrize("nh,nkv,hd,rot,bs", [(12, 2, 128, 128, 16), (6, 1, 48, 48, 16), (3, 3, 32, 16, 8),
                                              (5, 1, 64, 32, 32), (7, 1, 24, 16, 4), (4, 2, 40, 0, 16)])
@pytest.mark.parametrize("with_bias", [False, True])
def test_rope_kv_write_of_many_rows(nh, nkv, hd, rot, bs, with_bias):
    """A hundred and more rows of five sequences: portions that begin at a page's first slot, in its
    middle and at its last slot, a sequence of one token; against the float64 rotation, and bit for bit
    against the same rows sent 50 at a time (no slot beside the rows' own may change)."""
    torch.manual_seed(5)
    theta = 50000.0
    starts, counts = [0, 5, bs - 1, 3 * bs, 40], [45, 38, 2 * bs + 3, 1, 29]
    positions, tok_seq = [], []
    for s, (first, n) in enumerate(zip(starts, counts)):
        positions += list(range(first, first + n))
        tok_seq += [s] * n
    T = len(positions)
    assert T >= 64 and T % 16 != 0
    num_blocks = sum(-(-(a + n) // bs) for a, n in zip(starts, counts)) + 5
    tables = scattered_tables([a + n for a, n in zip(starts, counts)], bs, num_blocks, seed=4)
    qkv = torch.randn(T, (nh + 2 * nkv) * hd).bfloat16()
    pos_d = torch.tensor(positions, dtype=torch.int32, device=DEV)
    seq_d = torch.tensor(tok_seq, dtype=torch.int32, device=DEV)
    table = K().rope_table(pos_d, plain.rope_inv_freq(rot, theta).to(DEV)) if rot else None
    kp = torch.full((num_blocks, nkv, bs, hd), 7.0, dtype=torch.bfloat16)
    vp = torch.full((num_blocks, nkv, hd, bs), 7.0, dtype=torch.bfloat16)
    bias = torch.randn((nh + 2 * nkv) * hd).bfloat16() if with_bias else None
    d_bias = bias.to(DEV) if with_bias else None
    d_qkv, d_kp, d_vp = qkv.to(DEV), kp.to(DEV), vp.to(DEV)
    K().rope_kv_write(d_qkv, nh, nkv, hd, rot, table, pos_d, seq_d, tables.to(DEV), bs, d_kp, d_vp, d_bias)
    # the same rows, 50 at a time
    o_qkv, o_kp, o_vp = qkv.to(DEV), kp.to(DEV), vp.to(DEV)
    for first in range(0, T, 50):
        rows = slice(first, min(T, first + 50))
        K().rope_kv_write(o_qkv[rows], nh, nkv, hd, rot, table[rows] if rot else None, pos_d[rows], seq_d[rows],
                          tables.to(DEV), bs, o_kp, o_vp, d_bias)
    assert torch.equal(d_qkv, o_qkv) and torch.equal(d_kp, o_kp) and torch.equal(d_vp, o_vp)
    ref = (qkv.float() + bias.float()).bfloat16() if with_bias else qkv
    x = ref.double().view(T, nh + 2 * nkv, hd)
    rotated = x.clone()
    if rot:
        cos, sin = plain.rope_cos_sin(plain.rope_inv_freq(rot, theta, torch.float64), torch.tensor(positions), torch.float64)
        rotated[..., :rot] = x[..., :rot] * cos[:, None] + plain.rotate_half(x[..., :rot]) * sin[:, None]
    bound = tol("bfloat16", 4.0)
    assert (d_qkv.cpu().double().view(T, nh + 2 * nkv, hd)[:, :nh] - rotated[:, :nh]).abs().max() <= bound
    want_k, want_v = kp.clone().double(), vp.clone().double()
    untouched_k = torch.ones(num_blocks, bs, dtype=torch.bool)
    for t, (p, s) in enumerate(zip(positions, tok_seq)):
        blk = int(tables[s, p // bs])
        want_k[blk, :, p % bs, :] = rotated[t, nh:nh + nkv]
        want_v[blk, :, :, p % bs] = x[t, nh + nkv:]
        untouched_k[blk, p % bs] = False
    assert (d_kp.cpu().double() - want_k).abs().max() <= bound
    assert torch.equal(d_vp.cpu().double(), want_v)  # also: no slot beside the rows' own was written
    assert torch.equal(d_kp.cpu().permute(0, 2, 1, 3)[untouched_k], kp.permute(0, 2, 1, 3)[untouched_k])


@pytest.mark.parametrize("M", [1, 7, 16, 23, 64])
@pytest.mark.parametrize("nh,nkv,hd,rot,bs,Kdim,bias", [
    (4, 2, 16, 16, 4, 72, True), (6, 1, 48, 48, 16, 136, False), (3, 3, 32, 16, 8, 264, True),
    (5, 1, 64, 0, 16, 200, True), (12, 2, 128, 128, 16, 1536, True), (248, 4, 128, 64, 16, 136, True)])
@pytest.mark.parametrize("k_ranges", ["one", "chosen", "several"])
def test_gemm_skinny_rope(M, nh, nkv, hd, rot, bs, Kdim, bias, k_ranges):
    """The projection with rotation and cache write in its epilogue against: a float64 product,
    rounded to bfloat16 (as the separate projection would), rotated, and laid into the pools.
    With several k ranges the kernel adds up its workgroups' partial sums itself."""
    torch.manual_seed(M + nh)
    splits = {"one": 1, "chosen": None, "several": min(3, -(-Kdim // 128))}[k_ranges]
    theta = 50000.0
    # three sequences take turns; positions grow by 3 per row so that rows land in different pages
    tok_seq = [t % 3 for t in range(M)]
    positions = [2 + 3 * (t // 3) + 11 * (t % 3) for t in range(M)]
    lens = [max([p for p, s in zip(positions, tok_seq) if s == q] + [0]) + 1 for q in range(3)]
    num_blocks = sum(-(-n // bs) for n in lens) + 3
    tables = scattered_tables(lens, bs, num_blocks, seed=5)
    N = (nh + 2 * nkv) * hd
    a = (torch.randn(M, Kdim) * 0.5).to(torch.bfloat16)
    w = (torch.randn(N, Kdim) * 0.1).to(torch.bfloat16)
    b = torch.randn(N).to(torch.bfloat16) if bias else None
    kp = torch.full((num_blocks, nkv, bs, hd), 7.0, dtype=torch.bfloat16)
    vp = torch.full((num_blocks, nkv, hd, bs), 7.0, dtype=torch.bfloat16)
    d_kp, d_vp = kp.to(DEV), vp.to(DEV)
    q = torch.full((M, nh * hd), 9.0, dtype=torch.bfloat16, device=DEV)
    inv = (K().rope_table(torch.tensor(positions, dtype=torch.int32, device=DEV), plain.rope_inv_freq(rot, theta).to(DEV))
           if rot else None)
    K().gemm_skinny_rope(q, a.to(DEV), w.to(DEV), None if b is None else b.to(DEV), nh, nkv, hd, rot, inv,
                         torch.tensor(positions, dtype=torch.int32, device=DEV),
                         torch.tensor(tok_seq, dtype=torch.int32, device=DEV), tables.to(DEV), bs, d_kp, d_vp, splits)
    assert int(K().skinny_tickets(DEV).abs().sum()) == 0  # the tickets are back at zero
    exact = a.double() @ w.double().t() + (0 if b is None else b.double())
    x = exact.to(torch.bfloat16).double().view(M, nh + 2 * nkv, hd)
    rotated = x.clone()
    if rot:
        cos, sin = plain.rope_cos_sin(plain.rope_inv_freq(rot, theta, torch.float64), torch.tensor(positions),
                                      torch.float64)
        rotated[..., :rot] = x[..., :rot] * cos[:, None] + plain.rotate_half(x[..., :rot]) * sin[:, None]
    # one bfloat16 rounding of the product (values up to ~4 here) and one of the rotated value
    bound = 2.0 ** -8 * max(1.0, float(exact.abs().max())) * 2.5
    assert (q.cpu().double().view(M, nh, hd) - rotated[:, :nh]).abs().max() <= bound
    want_k, want_v = kp.clone().double(), vp.clone().double()
    touched = torch.zeros(num_blocks, dtype=torch.bool)
    for t, (p, s) in enumerate(zip(positions, tok_seq)):
        blk = int(tables[s, p // bs])
        touched[blk] = True
        want_k[blk, :, p % bs, :] = rotated[t, nh:nh + nkv]
        want_v[blk, :, :, p % bs] = x[t, nh + nkv:]
    assert (d_kp.cpu().double() - want_k).abs().max() <= bound
    assert (d_vp.cpu().double() - want_v).abs().max() <= bound
    # other pages keep what they held (other slots of touched pages are held to 7.0 by the bounds above)
    assert torch.equal(d_kp.cpu()[~touched], kp[~touched]) and torch.equal(d_vp.cpu()[~touched], vp[~touched])
    # queries only (a layer that reads another layer's cache): nothing is stored
    q2 = torch.empty_like(q)
    K().gemm_skinny_rope(q2, a.to(DEV), w[:nh * hd].contiguous().to(DEV), None if b is None else b[:nh * hd].to(DEV),
                         nh, 0, hd, rot, inv, torch.tensor(positions, dtype=torch.int32, device=DEV), None, None, bs,
                         None, None, splits)
    # (bit for bit where both calls take the same kernel and k ranges; the many-row kernel adds in another order)
    assert (q2.double() - q.double()).abs().max().item() <= (0.0 if N < 32768 and splits is not None else bound)


# ------------------------------------------------------------------ attention
def run_attention(kind, dtype, nh, nkv, hd, bs, window, seq_lens, q_lens, sharp=None, seed=0, ramp=None,
                  holes=False):
    """Queries are the last q_lens[s] positions of each sequence.  Returns (got, want).

    `sharp`: a key position of sequence 0 that dominates the scores of its last query, or
    (key position, index of the query within sequence 0's run).  `holes`: the pages of sequence 0
    that lie wholly before its first query's window are given back (their table entries are -1),
    and page 0 of the pool, which a kernel that follows a hole would land on, holds large values."""
    torch.manual_seed(seed)
    num_blocks = sum(-(-n // bs) for n in seq_lens) + 5
    tables = scattered_tables(seq_lens, bs, num_blocks, seed=seed + 1)
    if holes:
        assert window
        used = set(tables.flatten().tolist()) - {-1}
        if 0 in used:  # keep page 0 for the poison
            tables[tables == 0] = next(b for b in range(num_blocks) if b not in used)
        passed = max(0, seq_lens[0] - q_lens[0] - window + 1) // bs
        tables[0, :passed] = -1
    keys = [torch.randn(n, nkv, hd) for n in seq_lens]
    values = [torch.randn(n, nkv, hd) for n in seq_lens]
    positions, tok_seq = [], []
    for s, (n, ql) in enumerate(zip(seq_lens, q_lens)):
        positions += list(range(n - ql, n))
        tok_seq += [s] * ql
    T = len(positions)
    q = torch.randn(T, nh, hd)
    if sharp is not None:  # make one key of sequence 0 dominate the scores of one of its queries
        key_pos, q_index = sharp if isinstance(sharp, tuple) else (sharp, q_lens[0] - 1)
        direction = torch.randn(hd)
        direction /= direction.norm()
        keys[0][key_pos] = 6.0 * direction * math.sqrt(hd) ** 0.5
        q[q_index] = 6.0 * direction * math.sqrt(hd) ** 0.5
    if ramp is not None:  # scores of sequence 0 climb by `ramp` (natural-log units) per key, up or down
        direction = torch.randn(hd)
        direction /= direction.norm()
        keys[0] += (ramp * torch.arange(seq_lens[0]).float())[:, None, None] * direction * math.sqrt(hd) ** 0.5
        q[:q_lens[0]] += direction * math.sqrt(hd) ** 0.5
    scale = hd ** -0.5
    q, keys, values = q.to(DT[dtype]), [k.to(DT[dtype]) for k in keys], [v.to(DT[dtype]) for v in values]
    want = torch.stack([reference_attention(q[t].float(), keys[s].float(), values[s].float(), p, scale, window)
                        for t, (p, s) in enumerate(zip(positions, tok_seq))]).view(T, nh * hd)
    kp, vp = fill_pools(keys, values, tables, bs, num_blocks, DT[dtype])
    if holes:
        kp[0], vp[0] = 3.0e4, -3.0e4
    d = lambda x, dt=None: (x if dt is None else torch.tensor(x, dtype=dt)).to(DEV)
    out = torch.zeros(T, nh * hd, dtype=DT[dtype], device=DEV)
    qd = d(q.view(T, nh * hd).contiguous())
    pos_d, seq_d, tab_d = d(positions, torch.int32), d(tok_seq, torch.int32), d(tables)
    if kind == "generic":
        K().paged_attention_generic(out, qd, d(kp), d(vp), pos_d, seq_d, tab_d, nh, nkv, hd, scale, window)
    else:
        starts = [sum(q_lens[:s]) for s in range(len(q_lens))]
        dec = [[starts[s], positions[starts[s]], s, 0] for s in range(len(q_lens)) if q_lens[s] == 1]
        tiles = []
        for s, ql in enumerate(q_lens):
            if ql > 1:
                for first in range(0, ql, K().PREFILL_TILE):
                    tiles.append([s, starts[s] + first, min(K().PREFILL_TILE, ql - first)])
        if dec:
            K().attn_decode(out, qd, d(kp), d(vp), d(dec, torch.int32), tab_d, nh, nkv, hd, scale, window)
        if tiles:
            K().attn_prefill(out, qd, d(kp), d(vp), d(tiles, torch.int32), pos_d, tab_d, nh, nkv, hd, scale, window)
    return out.double().cpu(), want


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,bs,window", [(4, 2, 16, 4, 0), (6, 2, 48, 16, 0), (7, 1, 80, 8, 0),
                                                   (8, 8, 128, 16, 0), (6, 2, 64, 16, 37), (2, 1, 256, 32, 70)])
def test_generic_attention(dtype, nh, nkv, hd, bs, window):
    got, want = run_attention("generic", dtype, nh, nkv, hd, bs, window, [150, 1, 67, 330], [20, 1, 1, 75])
    assert (got - want).abs().max() <= (1e-5 if dtype == "float32" else 3e-2)


MFMA_SHAPES = [(12, 2, 128, 16, 0), (14, 2, 64, 16, 0), (4, 4, 32, 16, 0), (16, 1, 96, 32, 0),
               (7, 1, 256, 16, 0), (12, 2, 128, 16, 100), (6, 3, 64, 32, 33), (5, 1, 160, 16, 0)]


@pytest.mark.parametrize("nh,nkv,hd,bs,window", MFMA_SHAPES)
def test_matrix_core_attention_mixed_batch(nh, nkv, hd, bs, window):
    # decodes at an odd context, at one token, right after and right before a page's and a split's edge,
    # beside prompt portions of 2, 33 and 150 tokens (the last one starting in the middle of a cache)
    seq_lens = [777, 1, 257, 256, 40, 33, 600, 513]
    q_lens = [1, 1, 1, 1, 2, 33, 150, 1]
    got, want = run_attention("mfma", "bfloat16", nh, nkv, hd, bs, window, seq_lens, q_lens)
    err = (got - want).abs().max(dim=1).values
    assert float(err.max()) <= 3e-2, f"worst rows: {torch.topk(err, 5)}"


@pytest.mark.parametrize("kind", ["generic", "mfma"])
@pytest.mark.parametrize("key_pos,window,seen", [(3, 0, True), (255, 0, True), (256, 0, True), (700, 0, True),
                                                  (1299, 0, True), (1299 - 63, 64, True), (1299 - 64, 64, False)])
def test_one_far_key_stands_out(kind, key_pos, window, seen):
    """A single key carries almost all of the last query's weight: the output is that key's value
    if and only if the key is visible (far away among 1,300, on a page's or split's edge, at the
    window's edge), which a kernel that drops or adds one key cannot get right."""
    nh, nkv, hd, bs = 12, 2, 128, 16
    got, want = run_attention(kind, "bfloat16", nh, nkv, hd, bs, window, [1300, 90], [1, 1], sharp=key_pos)
    assert (got - want).abs().max() <= 3e-2
    # the construction works: the visible key really dominates (else the check above says little)
    if seen:
        assert want[0].abs().max() > 0.5


@pytest.mark.parametrize("kind", ["generic", "mfma"])
@pytest.mark.parametrize("q_len", [1, 2, 33, 64, 65])
@pytest.mark.parametrize("which", ["first", "last"])
@pytest.mark.parametrize("edge", ["before", "at", "unit"])
def test_window_edges_and_given_back_pages_in_runs(kind, q_len, which, edge):
    """A run of tokens over a window of 64 keys whose earlier pages have been given back (table
    entries of -1; page 0 of the pool holds large numbers).  One key dominates the scores of the
    run's first or last query: the key just before that query's window (which it must not see), the
    first key inside it, or a key on an edge of the 32-key units the matrix-core kernel walks.  The
    output is the plain one either way; one key too many or too few, or a read through a hole,
    gives something far from it."""
    nh, nkv, hd, bs, window, n = 12, 2, 128, 16, 64, 1300
    q_index = 0 if which == "first" else q_len - 1
    pos = n - q_len + q_index
    start = pos - window + 1
    key_pos = {"before": start - 1, "at": start, "unit": max(start, pos // 32 * 32)}[edge]
    got, want = run_attention(kind, "bfloat16", nh, nkv, hd, bs, window, [n, 90], [q_len, 1],
                              sharp=(key_pos, q_index), holes=True)
    assert torch.isfinite(got).all()
    assert (got - want).abs().max() <= 3e-2
    if edge != "before":  # the construction works: the output is nearly that key's value
        assert want[q_index].abs().max() > 0.5


@pytest.mark.parametrize("q_len", [2, 31, 32, 33, 64, 65, 100, 128, 129, 300])
def test_matrix_core_prefill_from_empty_and_warm(q_len):
    got, want = run_attention("mfma", "bfloat16", 12, 2, 128, 16, 0, [q_len, 200 + q_len], [q_len, q_len])
    assert (got - want).abs().max() <= 3e-2


@pytest.mark.parametrize("ramp", [0.02, 0.15, 0.5, -0.15])
def test_matrix_core_prefill_rising_scores(ramp):
    """The prefill kernel rescales its sums only when a score passes the running reference by 2^8:
    scores that climb slowly (never rescaled, weights grow to the limit), quickly (rescaled in
    nearly every 32 keys) or fall must all give the plain softmax."""
    got, want = run_attention("mfma", "bfloat16", 6, 2, 128, 16, 0, [700, 50], [700, 50], ramp=ramp)
    err = (got - want).abs().max(dim=1).values
    assert float(err.max()) <= 3e-2, f"worst rows: {torch.topk(err, 5)}"


@pytest.mark.parametrize("nh,nkv,hd,bs,window", MFMA_SHAPES)
def test_matrix_core_long_prefill_shapes(nh, nkv, hd, bs, window):
    got, want = run_attention("mfma", "bfloat16", nh, nkv, hd, bs, window, [333, 700, 130], [333, 190, 77])
    err = (got - want).abs().max(dim=1).values
    assert float(err.max()) <= 3e-2, f"worst rows: {torch.topk(err, 5)}"


# ------------------------------------------------------------------ sampling
def test_argmax_ties_across_chunks():
    """A vocabulary of many chunks, the maximum tied between chunks: the first index wins
    (torch.argmax's rule, which the reference's greedy path relies on)."""
    V = 70001
    logits = torch.randn(5, V)
    logits[0, [69000, 1500, 30000]] = 50.0
    logits[1, [V - 1, V - 2]] = 50.0
    logits[2, 0] = 50.0
    logits[3, :] = 1.25           # everything tied
    logits[4, [40000, 40001]] = 50.0
    tokens = torch.empty(5, dtype=torch.int32, device=DEV)
    K().sample(tokens, logits.to(DEV), None, None)
    assert tokens.cpu().tolist() == [1500, V - 2, 0, 0, 40000]
    K().sample(tokens, logits.to(DEV), torch.zeros(5, device=DEV), torch.rand(5, device=DEV))
    assert tokens.cpu().tolist() == [1500, V - 2, 0, 0, 40000]


def test_sampling_kernel():
    torch.manual_seed(5)
    V = 1000
    logits = torch.randn(6, V) * 2
    logits[1, 400] = logits[1, 17] = 9.0  # a tie: the first maximum wins
    logits[2] = -1e9
    logits[2, 777] = 0.0                 # one-hot
    temps = torch.tensor([0.0, 0.0, 0.8, 0.8, 1.5, 0.3])
    us = torch.tensor([0.3, 0.9, 0.99, 0.5, 0.123, 0.77])
    tokens = torch.empty(6, dtype=torch.int32, device=DEV)
    K().sample(tokens, logits.to(DEV), temps.to(DEV), us.to(DEV))
    got = tokens.cpu().tolist()
    want = [plain.sample_from_logits(logits[r], float(temps[r]), float(us[r])) for r in range(6)]
    assert got == want and got[1] == 17 and got[2] == 777
    K().sample(tokens, logits.to(DEV), None, None)
    assert tokens.cpu().tolist() == logits.argmax(-1).tolist()
    # a wide vocabulary that is no multiple of the block, many draws
    V = 151_936 + 3
    row = torch.randn(1, V) * 3
    d_row = row.to(DEV)
    for u in (0.0, 1e-7, 0.25, 0.5, 0.75, 0.999999):
        K().sample(tokens[:1], d_row, torch.tensor([0.9], device=DEV), torch.tensor([u], device=DEV))
        assert int(tokens[0]) == plain.sample_from_logits(row[0], 0.9, u)
