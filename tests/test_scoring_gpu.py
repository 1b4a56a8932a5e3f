"""GPU parity tests of the scoring path (fp32 MFMA GEMMs + SPD inverse) against the float64
oracle.  Tolerance: 1e-4 relative (to the largest magnitude of the result) as stated for the
scores; GEMMs alone are held to the fp32 accumulation bound 1e-6 + 2e-7*sqrt(K)."""
import math

import numpy as np
import pytest
import torch

from oracle import score_oracle as so
import trak_amd.score_computers as score_computers_module
from trak_amd import _lib
import trak_amd.utils as utils_module
from trak_amd import BasicScoreComputer, get_matrix_mult
from trak_amd.utils import (
    gemm_nt,
    gemm_nt16,
    gemm_nt_split,
    gemm_tn,
    gram_split,
    matmul_nt,
    spd_inverse,
    split2_rows,
    split_rows,
)

pytestmark = pytest.mark.gpu


def gemm_tol(K):
    return 1e-6 + 2e-7 * math.sqrt(K)


def rel_max(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return np.abs(got - want).max() / max(np.abs(want).max(), 1e-300)


@pytest.mark.parametrize("M,N,K", [(128, 128, 16), (256, 384, 64), (1, 1, 1), (130, 70, 33), (1000, 513, 257), (64, 2048, 4096)])
def test_gemm_nt(gpu, M, N, K):
    gen = torch.Generator(device="cpu").manual_seed(M * 7 + N)
    a, b = torch.randn(M, K, generator=gen), torch.randn(N, K, generator=gen)
    want = a.double().numpy() @ b.double().numpy().T
    got = gemm_nt(a.to(gpu), b.to(gpu))
    assert got.shape == (M, N) and rel_max(got.cpu().numpy(), want) < gemm_tol(K)
    # alpha, beta and the row scale epilogue
    c0 = torch.randn(M, N, generator=gen)
    rs = torch.rand(M, generator=gen)
    got = gemm_nt(a.to(gpu), b.to(gpu), out=c0.clone().to(gpu), alpha=0.5, beta=-2.0, row_scale=rs.to(gpu))
    want2 = (0.5 * want - 2.0 * c0.double().numpy()) * rs.double().numpy()[:, None]
    assert rel_max(got.cpu().numpy(), want2) < gemm_tol(K)


@pytest.mark.parametrize("M,N,K", [(130, 70, 40), (300, 515, 128), (129, 1, 8), (2100, 2050, 128), (4000, 3000, 120)])
def test_gemm_nt_short_contraction(gpu, M, N, K):
    """K <= 128 in multiples of 8 with aligned rows takes the kernel that holds both operand tiles
    whole (up to 512 tiles); ragged edges, accumulation into C, and the hand-over to the general
    kernel above that tile count."""
    gen = torch.Generator(device="cpu").manual_seed(M + 3 * N + K)
    a, b = torch.randn(M, K, generator=gen), torch.randn(N, K, generator=gen)
    c0 = torch.randn(M, N, generator=gen)
    want = a.double().numpy() @ b.double().numpy().T
    got = gemm_nt(a.to(gpu), b.to(gpu))
    assert rel_max(got.cpu().numpy(), want) < gemm_tol(K)
    got = gemm_nt(a.to(gpu), b.to(gpu), out=c0.clone().to(gpu), alpha=-1.0, beta=1.0)
    assert rel_max(got.cpu().numpy(), c0.double().numpy() - want) < gemm_tol(K)
    # a padded destination keeps its padding
    wide = torch.full((M, N + 5), 7.0, device=gpu)
    gemm_nt(a.to(gpu), b.to(gpu), out=wide[:, :N])
    assert rel_max(wide[:, :N].cpu().numpy(), want) < gemm_tol(K) and bool((wide[:, N:] == 7.0).all())


@pytest.mark.parametrize("M,N,K", [(128, 128, 16), (96, 200, 1000), (33, 17, 5), (512, 512, 2050)])
def test_gemm_tn(gpu, M, N, K):
    gen = torch.Generator(device="cpu").manual_seed(M + N + K)
    a, b = torch.randn(K, M, generator=gen), torch.randn(K, N, generator=gen)
    want = a.double().numpy().T @ b.double().numpy()
    got = gemm_tn(a.to(gpu), b.to(gpu))
    assert rel_max(got.cpu().numpy(), want) < gemm_tol(K)
    acc = gemm_tn(a.to(gpu), b.to(gpu), out=got.clone(), beta=1.0)
    assert rel_max(acc.cpu().numpy(), 2 * want) < gemm_tol(K)


def test_gemm_on_strided_views(gpu):
    gen = torch.Generator(device="cpu").manual_seed(3)
    big_a, big_b = torch.randn(300, 200, generator=gen).to(gpu), torch.randn(150, 200, generator=gen).to(gpu)
    a, b = big_a[10:210, 3:131], big_b[5:105, 3:131]           # unaligned start, pitch 200
    out = torch.zeros(256, 160, device=gpu)
    gemm_nt(a, b, out=out[20:220, 7:107])
    want = a.double().cpu().numpy() @ b.double().cpu().numpy().T
    assert rel_max(out[20:220, 7:107].cpu().numpy(), want) < gemm_tol(128)
    assert out[:20].abs().max() == 0 and out[:, :7].abs().max() == 0 and out[:, 107:].abs().max() == 0


@pytest.mark.parametrize("n,lam", [(128, 0.0), (100, 0.5), (384, 1e-3), (513, 0.0), (1000, 1e-3)])
def test_spd_inverse(gpu, n, lam):
    gen = torch.Generator(device="cpu").manual_seed(n)
    x = torch.randn(3 * n, n, generator=gen) / math.sqrt(n)
    a = (x.T @ x).contiguous()
    a = (a + a.T) / 2
    want = np.linalg.inv(a.double().numpy() + lam * np.eye(n))
    inv, mean_abs = spd_inverse(a.to(gpu), lambda_reg=lam, normalize=False)
    assert rel_max(inv.cpu().numpy(), want) < 1e-4
    assert abs(mean_abs.item() - np.abs(want).mean()) / np.abs(want).mean() < 1e-4
    invn, m2 = spd_inverse(a.to(gpu), lambda_reg=lam, normalize=True)
    assert rel_max(invn.cpu().numpy(), want / np.abs(want).mean()) < 1e-4
    assert torch.equal(m2, mean_abs)
    # (A + lambda I) inv = I
    prod = (a.double().numpy() + lam * np.eye(n)) @ inv.double().cpu().numpy()
    assert np.abs(prod - np.eye(n)).max() < 1e-3


def test_spd_inverse_many_blocks(gpu):
    # 67 diagonal blocks: more tree nodes of one shape than one batched launch takes, odd block counts
    n, lam = 8500, 1e-2
    gen = torch.Generator(device=gpu).manual_seed(8500)
    X = torch.randn(3 * n, n, generator=gen, device=gpu) / math.sqrt(n)
    a = (X.double().T @ X.double()).float()
    inv, mean_abs = spd_inverse(a, lambda_reg=lam, normalize=True)
    a64 = a.double() + lam * torch.eye(n, device=gpu, dtype=torch.float64)
    resid = a64 @ (inv.double() * mean_abs.double()) - torch.eye(n, device=gpu, dtype=torch.float64)
    assert float(resid.abs().max()) < 1e-4
    assert float((inv - inv.T).abs().max()) <= 1e-5 * float(inv.abs().max())


def test_spd_inverse_closed_forms_and_failure(gpu):
    d = torch.arange(1, 201, dtype=torch.float32)
    inv, _ = spd_inverse(torch.diag(d * d).to(gpu), lambda_reg=0.5)
    assert torch.allclose(inv.diagonal().cpu(), 1.0 / (d * d + 0.5), rtol=1e-6)
    assert (inv - torch.diag(inv.diagonal())).abs().max() == 0
    ident, m = spd_inverse(torch.eye(300, device=gpu), lambda_reg=1.0, normalize=True)
    assert torch.allclose(ident, torch.eye(300, device=gpu) * 300.0)        # (I/2) / mean|I/2|
    assert abs(m.item() - 0.5 / 300) < 1e-9
    bad = torch.eye(140)
    bad[130, 130] = -1.0
    with pytest.raises(torch.linalg.LinAlgError):
        spd_inverse(bad.to(gpu))


def test_gram_matrices_that_are_not_positive_definite(gpu):
    # The reference inverts with LU (trak/score_computers.py:163), which returns something for every
    # matrix that is not exactly singular; the Cholesky path needs a positive definite matrix.
    from trak_amd import BasicScoreComputer

    gen = torch.Generator().manual_seed(3)
    # (1) fewer training points than proj_dim, ridge > 0: rank-deficient Gram + lambda I is positive
    #     definite, and the inverse must match float64
    N, k, lam = 60, 256, 1e-2
    X = torch.randn(N, k, generator=gen) / 8
    sc = BasicScoreComputer(dtype=torch.float32, device=gpu, lambda_reg=lam)
    xtx = sc.get_xtx(X.to(gpu))
    feats = sc.get_x_xtx_inv(X.to(gpu), xtx).cpu().numpy().astype(np.float64)
    x64 = X.numpy().astype(np.float64)
    inv64 = np.linalg.inv(x64.T @ x64 + lam * np.eye(k))
    want = x64 @ (inv64 / np.abs(inv64).mean())
    # X lies in the span where the inverse is small (1/9 .. 1) while the inverse itself is dominated by
    # 1/lambda = 100 on the complement: X @ inv cancels two orders of magnitude, so fp32 arithmetic
    # (this library's or torch.linalg.inv's alike) gives these features to about 1e-4, not 1e-6
    err = np.abs(feats - want).max() / np.abs(want).max()
    ref = torch.linalg.inv(xtx.double().cpu().float() + lam * torch.eye(k))
    ref_err = np.abs((X @ (ref / ref.abs().mean())).numpy() - want).max() / np.abs(want).max()
    assert err < max(1e-3, 3 * ref_err)
    # (2) the same with lambda_reg = 0 (TRAKer's default): the Gram matrix is singular up to rounding.
    #     The Cholesky path fails and the pivoted elimination answers, as the reference's LU does,
    #     or raises LinAlgError when it meets a zero pivot - never anything else
    sc0 = BasicScoreComputer(dtype=torch.float32, device=gpu, lambda_reg=0.0)
    #     (the inverse of a numerically singular matrix is rounding noise, so there are no values to compare)
    try:
        f0 = sc0.get_x_xtx_inv(X.to(gpu), xtx)
        assert f0.shape == (N, k)
    except torch.linalg.LinAlgError:
        pass
    # (3) an ill-conditioned Gram matrix rounded to fp16 (TRAKer's use_half_precision default hands the
    #     inverse exactly this): the rounding makes it indefinite.  The result must be the inverse of the
    #     matrix that was handed over, as the reference's LU gives it
    k = 192
    q, _ = torch.linalg.qr(torch.randn(k, k, generator=gen, dtype=torch.float64))
    spectrum = 1000.0 / torch.arange(1, k + 1, dtype=torch.float64) ** 2.5      # condition number 5e5
    gram = ((q * spectrum) @ q.T).half()
    g64 = gram.double().numpy()
    assert np.linalg.eigvalsh((g64 + g64.T) / 2).min() < 0                       # indefinite after the rounding
    with pytest.raises(torch.linalg.LinAlgError):
        spd_inverse(gram.float().to(gpu))
    inv, mean_abs = spd_inverse(gram.float().to(gpu), normalize=True, general_fallback=True)
    # two backward-stable eliminations of a matrix with condition number 5e5 agree with the exact inverse
    # (and with each other) to about condition number x 2^-24, no closer: the yardstick is the error of the
    # reference's own call, torch.linalg.inv, on the same fp32 matrix
    inv64 = np.linalg.inv(g64)
    ref = torch.linalg.inv(gram.float().to(gpu)).double().cpu().numpy()
    got = (inv.double() * mean_abs.double()).cpu().numpy()
    scale = np.abs(inv64).max()
    err, ref_err = np.abs(got - inv64).max() / scale, np.abs(ref - inv64).max() / scale
    print("general inverse error", err, "torch.linalg.inv error", ref_err)
    assert err < max(4 * ref_err, np.linalg.cond(g64) * 2.0**-24), (err, ref_err)
    assert abs(mean_abs.item() - np.abs(got).mean()) <= 1e-5 * np.abs(got).mean()
    resid = np.abs(g64 @ got - np.eye(k)).max()
    assert resid < max(4 * np.abs(g64 @ ref - np.eye(k)).max(), 1e-3), resid
    sch = BasicScoreComputer(dtype=torch.float16, device=gpu, lambda_reg=0.0)
    Xh = (torch.randn(500, k, generator=gen) / 8).half().to(gpu)
    out = sch.get_x_xtx_inv(Xh, gram.to(gpu))
    assert out.dtype == torch.float16 and torch.isfinite(out).all()


# (up to 2944 every elimination step goes over the whole matrix; from 3072 on the steps run inside blocks of 64
# columns; above 6144 the panels are 8 columns wide instead of 16)
@pytest.mark.parametrize("n", [1, 5, 16, 100, 128, 129, 300, 1000, 2048, 3100, 6200])
def test_general_inverse_against_float64(gpu, n):
    # nonsymmetric, indefinite, well conditioned: inverse to fp32 accuracy, A * inv = I
    from trak_amd.utils import general_inverse

    gen = torch.Generator().manual_seed(n)
    a = torch.randn(n, n, generator=gen) / math.sqrt(n) + torch.diag(torch.where(torch.rand(n, generator=gen) < 0.5, -2.0, 2.0))
    inv, mean_abs = general_inverse(a.to(gpu), lambda_reg=0.25)
    a64 = a.double().numpy() + 0.25 * np.eye(n)
    want = np.linalg.inv(a64)
    got = inv.cpu().numpy().astype(np.float64)
    # (the condition number in the 2-norm, or for the large cases its cheaper bound through 1-norms)
    cond = np.linalg.cond(a64) if n <= 2048 else np.linalg.norm(a64, 1) * np.linalg.norm(want, 1)
    assert np.abs(got - want).max() <= 2e-5 * np.abs(want).max() * max(1.0, cond / 10)
    assert np.abs(a64 @ got - np.eye(n)).max() < 1e-4
    assert abs(mean_abs.item() - np.abs(got).mean()) <= 1e-5 * np.abs(got).mean()
    norm, _ = general_inverse(a.to(gpu), lambda_reg=0.25, normalize=True)
    assert torch.allclose(norm, inv / mean_abs, rtol=1e-6, atol=0)


def test_general_inverse_needs_its_pivoting(gpu):
    from trak_amd.utils import general_inverse

    # zeros on the diagonal: elimination without row exchanges would divide by zero at once
    n = 200
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(1))
    a = torch.zeros(n, n)
    a[torch.arange(n), perm] = torch.arange(1, n + 1, dtype=torch.float32)      # a scaled permutation matrix
    a[0, 0] = 0.0 if perm[0] != 0 else a[0, 0]
    inv, _ = general_inverse(a.to(gpu))
    assert torch.equal(inv.cpu(), torch.linalg.inv(a.double()).float())          # exact: one entry per row
    # pivots far below the diagonal block of a step, and rows that are displaced more than once
    gen = torch.Generator().manual_seed(2)
    b = torch.randn(300, 300, generator=gen)
    b[:40] *= 1e-3                                 # the first rows are never the largest in their columns
    got, _ = general_inverse(b.to(gpu))
    want = np.linalg.inv(b.double().numpy())
    assert np.abs(got.cpu().numpy() - want).max() < 1e-3 * np.abs(want).max()
    # an exactly singular matrix: a zero pivot raises, as torch.linalg.inv does
    c = torch.randn(50, 50, generator=gen)
    c[:, 7] = 0.0
    with pytest.raises(torch.linalg.LinAlgError):
        general_inverse(c.to(gpu))
    with pytest.raises(torch.linalg.LinAlgError):
        torch.linalg.inv(c.to(gpu))


def test_general_inverse_in_column_blocks_needs_its_pivoting(gpu):
    # the same three situations at a size where the steps run inside blocks of 64 columns
    from trak_amd.utils import general_inverse

    n = 3300
    perm = torch.randperm(n, generator=torch.Generator().manual_seed(3))
    a = torch.zeros(n, n)
    a[torch.arange(n), perm] = 1.0 + torch.arange(n, dtype=torch.float32) / 1024    # a scaled permutation matrix
    inv, _ = general_inverse(a.to(gpu))
    assert torch.equal(inv.cpu(), torch.linalg.inv(a.double()).float())              # exact: one entry per row
    # pivots far below the block, rows displaced more than once within a block and from block to block
    gen = torch.Generator().manual_seed(4)
    b = torch.randn(n, n, generator=gen)
    b[:700] *= 1e-3
    got, _ = general_inverse(b.to(gpu))
    # condition number about 1e7: measured against what LAPACK's LU with the same pivoting makes of it in fp32
    b64 = b.double().numpy()
    want = np.linalg.inv(b64)
    ref = torch.linalg.inv(b).double().numpy()      # (on the CPU; numpy's inverse of an fp32 matrix computes in double)
    g64 = got.cpu().numpy().astype(np.float64)
    err, ref_err = (float(np.abs(m - want).max() / np.abs(want).max()) for m in (g64, ref))
    resid, ref_resid = (float(np.abs(b64 @ m - np.eye(n)).max()) for m in (g64, ref))
    assert err <= 4 * ref_err + 1e-5 and resid <= 2 * ref_resid + 1e-3, (err, ref_err, resid, ref_resid)
    # a zero column in the last panel of a block
    c = torch.randn(n, n, generator=gen)
    c[:, 3135] = 0.0
    with pytest.raises(torch.linalg.LinAlgError):
        general_inverse(c.to(gpu))


def test_general_inverse_of_an_indefinite_gram_matrix_at_proj_dim_4096(gpu):
    # the case the fallback exists for, at the benchmark's proj_dim: a Gram matrix rounded to fp16
    from trak_amd.utils import general_inverse

    k = 4096
    gen = torch.Generator(device=gpu).manual_seed(5)
    q, _ = torch.linalg.qr(torch.randn(k, k, generator=gen, device=gpu, dtype=torch.float64))
    spectrum = 1000.0 / torch.arange(1, k + 1, dtype=torch.float64, device=gpu) ** 1.5   # condition number 2.6e5
    gram = ((q * spectrum) @ q.T).half().float()    # the rounding noise exceeds the smallest eigenvalues
    with pytest.raises(torch.linalg.LinAlgError):
        spd_inverse(gram)
    inv, mean_abs = general_inverse(gram, normalize=True)
    assert torch.isfinite(inv).all()
    resid = (gram.double() @ (inv.double() * mean_abs.double()) - torch.eye(k, device=gpu, dtype=torch.float64)).abs().max()
    ref = torch.linalg.inv(gram.cpu()).to(gpu)      # LAPACK's LU in fp32 on the CPU, same pivoting: the size of the residual
    ref_resid = (gram.double() @ ref.double() - torch.eye(k, device=gpu, dtype=torch.float64)).abs().max()
    assert float(resid) < max(1e-2, 20 * float(ref_resid)), (float(resid), float(ref_resid))


def split_planes_to_numpy(op):
    """[planes, padded rows, padded K] float32 view of a SplitOperand (layout: plane, k-octet, row,
    8 values of 16 bits: bf16 for an fp32 or bf16 source, fp16 for an fp16 source)."""
    planes = 3 if op.dtype == torch.float32 else 1
    Rp, K8 = (op.rows + 255) // 256 * 256, (op.K + 63) // 64 * 8
    raw = op.planes.cpu().numpy()[: planes * K8 * Rp * 16].view(np.uint16).reshape(planes, K8, Rp, 8)
    if op.dtype == torch.float16:
        vals = raw.view(np.float16).astype(np.float32)
    else:
        vals = (raw.astype(np.uint32) << 16).view(np.float32)
    return vals.transpose(0, 2, 1, 3).reshape(planes, Rp, K8 * 8)


@pytest.mark.parametrize("rows,K,transposed", [(5, 9, False), (300, 70, False), (70, 300, True), (257, 33, True), (256, 16, False)])
def test_split_is_exact_and_zero_padded(gpu, rows, K, transposed):
    gen = torch.Generator(device="cpu").manual_seed(rows * K)
    t = torch.randn((K, rows) if transposed else (rows, K), generator=gen)
    t *= 10.0 ** torch.randint(-12, 12, t.shape, generator=gen).float()       # every binade in reach
    t.view(-1)[:3] = torch.tensor([0.0, -0.0, 1.0])
    wide = torch.zeros(t.shape[0], t.shape[1] + 3)
    wide[:, 1 : 1 + t.shape[1]] = t
    for src in (t.to(gpu), wide.to(gpu)[:, 1 : 1 + t.shape[1]]):               # aligned rows, then pitched unaligned rows
        op = split_rows(src, transposed=transposed)
        planes = split_planes_to_numpy(op).astype(np.float64)
        want = (t.T if transposed else t).numpy().astype(np.float64)
        total = planes[0] + planes[1] + planes[2]
        assert np.array_equal(total[:rows, :K], want)                          # three bf16 terms, exact sum
        assert not total[rows:].any() and not total[:, K:].any()               # padding rewritten as zeros
        nz = want != 0
        assert (np.abs(planes[1][:rows, :K][nz]) <= 2.0 ** -8 * np.abs(planes[0][:rows, :K][nz])).all()
        assert (np.abs(planes[2][:rows, :K][nz]) <= 2.0 ** -16 * np.abs(planes[0][:rows, :K][nz])).all()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("rows,K,transposed", [(5, 9, False), (300, 70, False), (70, 300, True), (257, 33, True), (256, 64, False)])
def test_sixteen_bit_operands_are_one_exact_plane(gpu, dtype, rows, K, transposed):
    gen = torch.Generator(device="cpu").manual_seed(rows + K)
    t = (torch.randn((K, rows) if transposed else (rows, K), generator=gen) * 3).to(dtype)
    wide = torch.zeros(t.shape[0], t.shape[1] + 3, dtype=dtype)
    wide[:, 1 : 1 + t.shape[1]] = t
    for src in (t.to(gpu), wide.to(gpu)[:, 1 : 1 + t.shape[1]]):
        op = split_rows(src, transposed=transposed)
        assert op.dtype == dtype
        planes = split_planes_to_numpy(op)
        want = (t.T if transposed else t).float().numpy()
        assert planes.shape[0] == 1 and np.array_equal(planes[0][:rows, :K], want)
        assert not planes[0][rows:].any() and not planes[0][:, K:].any()


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (130, 70, 33), (256, 512, 64), (1000, 513, 257), (300, 700, 4100)])
def test_gemm_nt_split_sixteen_bit(gpu, dtype, M, N, K):
    # products of 16-bit values are exact in fp32: the only error is the fp32 accumulation
    gen = torch.Generator(device="cpu").manual_seed(M + N * 3 + K)
    a, b = torch.randn(M, K, generator=gen).to(dtype), torch.randn(N, K, generator=gen).to(dtype)
    want = a.double().numpy() @ b.double().numpy().T
    sa, sb = split_rows(a.to(gpu)), split_rows(b.to(gpu))
    got = gemm_nt_split(sa, sb)
    assert rel_max(got.cpu().numpy(), want) < gemm_tol(K)
    # the same numbers through the three-plane fp32 path (the extra planes are zero)
    ref = gemm_nt_split(split_rows(a.float().to(gpu)), split_rows(b.float().to(gpu)))
    assert rel_max(got.cpu().numpy(), ref.cpu().numpy()) < gemm_tol(K)
    rs = torch.rand(M, generator=gen)
    c0 = torch.randn(M, N, generator=gen)
    got = gemm_nt_split(sa, sb, out=c0.clone().to(gpu), alpha=2.0, beta=0.5, row_scale=rs.to(gpu))
    assert rel_max(got.cpu().numpy(), (2.0 * want + 0.5 * c0.double().numpy()) * rs.double().numpy()[:, None]) < gemm_tol(K)
    g = gram_split(split_rows(a.T.contiguous().to(gpu), transposed=True))
    assert torch.equal(g, g.T) and rel_max(g.cpu().numpy(), a.double().numpy() @ a.double().numpy().T) < gemm_tol(K)
    with pytest.raises(RuntimeError):
        gemm_nt_split(sa, split_rows(b.float().to(gpu)))        # operands of different source types


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("M,N,K", [(1, 1, 64), (130, 70, 128), (256, 512, 64), (1000, 513, 256), (300, 700, 4096), (257, 255, 1088)])
def test_gemm_nt16_reads_operands_in_place(gpu, dtype, M, N, K):
    """The in-place 16-bit product issues the same MFMAs in the same order as the one-plane product,
    so the two agree bit for bit; ragged tiles, accumulation, row scale, operands that are column
    slices of wider buffers."""
    gen = torch.Generator(device="cpu").manual_seed(M + N * 3 + K)
    a, b = torch.randn(M, K, generator=gen).to(dtype), torch.randn(N, K, generator=gen).to(dtype)
    want = a.double().numpy() @ b.double().numpy().T
    ag, bg = a.to(gpu), b.to(gpu)
    got = gemm_nt16(ag, bg)
    assert got.dtype == torch.float32 and rel_max(got.cpu().numpy(), want) < gemm_tol(K)
    assert torch.equal(got, gemm_nt_split(split_rows(ag), split_rows(bg)))
    assert torch.equal(got, matmul_nt(ag, bg))
    rs = torch.rand(M, generator=gen)
    c0 = torch.randn(M, N, generator=gen)
    got = gemm_nt16(ag, bg, out=c0.clone().to(gpu), alpha=2.0, beta=0.5, row_scale=rs.to(gpu))
    assert rel_max(got.cpu().numpy(), (2.0 * want + 0.5 * c0.double().numpy()) * rs.double().numpy()[:, None]) < gemm_tol(K)
    # slices of wider buffers: pitch K + 24, first column 8 (rows stay 16-byte aligned)
    wa = torch.zeros(M, K + 24, dtype=dtype, device=gpu)
    wb = torch.zeros(N, K + 24, dtype=dtype, device=gpu)
    wa[:, 8:8 + K], wb[:, 8:8 + K] = ag, bg
    wide = torch.full((M, N + 3), -1.0, device=gpu)
    gemm_nt16(wa[:, 8:8 + K], wb[:, 8:8 + K], out=wide[:, :N])
    assert torch.equal(wide[:, :N], gemm_nt16(ag, bg)) and bool((wide[:, N:] == -1.0).all())


def test_gemm_nt16_refuses_what_it_cannot_read_in_place(gpu):
    a = torch.randn(64, 128, device=gpu).half()
    b = torch.randn(32, 128, device=gpu).half()
    with pytest.raises(RuntimeError):
        gemm_nt16(a[:, :100], b[:, :100])                    # K not a multiple of 64
    with pytest.raises(RuntimeError):
        gemm_nt16(a[:, 4:68], b[:, 4:68])                    # rows start 8 bytes off
    with pytest.raises(RuntimeError):
        gemm_nt16(a, b.bfloat16())                           # operands of different types
    with pytest.raises(RuntimeError):
        gemm_nt16(a.float(), b.float())
    # matmul_nt takes all of them (through planes)
    want = a[:, :100].double() @ b[:, :100].double().T
    assert rel_max(matmul_nt(a[:, :100], b[:, :100]).cpu().numpy(), want.cpu().numpy()) < gemm_tol(100)
    want = a[:, 4:68].double() @ b[:, 4:68].double().T
    assert rel_max(matmul_nt(a[:, 4:68], b[:, 4:68]).cpu().numpy(), want.cpu().numpy()) < gemm_tol(64)
    want = a.double() @ b.bfloat16().double().T
    assert rel_max(matmul_nt(a, b.bfloat16()).cpu().numpy(), want.cpu().numpy()) < gemm_tol(128)


def split2_planes_to_numpy(op):
    """[2, padded rows, padded K] float64 values of the two fp16 planes of a split2 operand."""
    Rp, K8 = (op.rows + 255) // 256 * 256, (op.K + 63) // 64 * 8
    raw = op.planes.cpu().numpy()[: 2 * K8 * Rp * 16].view(np.float16).reshape(2, K8, Rp, 8)
    return raw.astype(np.float64).transpose(0, 2, 1, 3).reshape(2, Rp, K8 * 8)


@pytest.mark.parametrize("rows,K,transposed", [(5, 9, False), (300, 70, False), (70, 300, True), (257, 33, True), (256, 64, False)])
def test_split2_rows_scales_and_planes(gpu, rows, K, transposed):
    """Two fp16 planes of the row-scaled operand: the row factor is the power of two that puts the
    row's largest magnitude into [2^14, 2^15); h1 + h2 equals the scaled value up to 2^-11 of the
    smaller term (2^-26 of the row's largest magnitude at worst); padding is zero."""
    gen = torch.Generator(device="cpu").manual_seed(rows * K + 1)
    t = torch.randn((rows, K), generator=gen)
    t *= (10.0 ** torch.randint(-20, 20, (rows, 1), generator=gen).float())      # rows of very different size
    t[0, :] = 0.0                                                              # a row of zeros
    if rows > 3:
        t[3, 1:] *= 1e-9                                                       # one large entry, the rest tiny
    src = (t.T.contiguous() if transposed else t).to(gpu)
    op = split2_rows(src, transposed=transposed)
    assert op.rows == rows and op.K == K and op.scales is not None
    planes = split2_planes_to_numpy(op)
    unscale = op.scales[:rows].cpu().double().numpy()
    amax = t.abs().max(dim=1).values.double().numpy()
    want_unscale = np.where(amax > 0, 2.0 ** (np.floor(np.log2(np.where(amax > 0, amax, 1.0))) - 14), 1.0)
    assert np.array_equal(unscale, want_unscale)
    scaled = t.double().numpy() / unscale[:, None]
    assert np.abs(scaled).max() < 2.0 ** 15
    got = planes[0, :rows, :K] + planes[1, :rows, :K]
    # h1 carries 11 bits; h2 the next 11 unless it is subnormal in fp16 (absolute error 2^-25 then)
    err = np.abs(got - scaled)
    assert np.all(err <= np.maximum(np.abs(scaled) * 2.0 ** -21, 2.0 ** -25))
    assert np.array_equal(planes[0, :rows, :K], scaled.astype(np.float16).astype(np.float64))   # RNE first term
    assert np.count_nonzero(planes[:, rows:, :]) == 0 and np.count_nonzero(planes[:, :, K:]) == 0


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (130, 70, 33), (256, 512, 64), (1000, 513, 257), (64, 2048, 4096), (129, 257, 8200)])
def test_gemm_nt_split2(gpu, M, N, K):
    """Three fp16 MFMAs on two planes per operand: error bounded by 2^-21 of sum |a||b| plus the fp32
    accumulation; alpha, beta, row scale; rows of very different magnitude keep their relative accuracy."""
    gen = torch.Generator(device="cpu").manual_seed(M + N * 3 + K + 2)
    a, b = torch.randn(M, K, generator=gen), torch.randn(N, K, generator=gen)
    a *= 10.0 ** torch.randint(-12, 12, (M, 1), generator=gen).float()
    b *= 10.0 ** torch.randint(-12, 12, (N, 1), generator=gen).float()
    a64, b64 = a.double().numpy(), b.double().numpy()
    want = a64 @ b64.T
    bound = np.abs(a64) @ np.abs(b64).T                       # sum |a||b| per entry
    sa, sb = split2_rows(a.to(gpu)), split2_rows(b.to(gpu))
    got = gemm_nt_split(sa, sb).cpu().double().numpy()
    assert np.all(np.abs(got - want) <= bound * (2.0 ** -20 + 2e-7 * math.sqrt(K)) + 1e-300)
    rs = torch.rand(M, generator=gen)
    c0 = torch.randn(M, N, generator=gen) * float(np.abs(want).max())
    got = gemm_nt_split(sa, sb, out=c0.clone().to(gpu), alpha=2.0, beta=0.5, row_scale=rs.to(gpu)).cpu().double().numpy()
    want2 = (2.0 * want + 0.5 * c0.double().numpy()) * rs.double().numpy()[:, None]
    tol = (2.0 * bound + 0.5 * np.abs(c0.double().numpy())) * (2.0 ** -20 + 2e-7 * math.sqrt(K)) + 1e-300
    assert np.all(np.abs(got - want2) <= tol)
    assert torch.equal(matmul_nt(a.to(gpu), b.to(gpu), two_planes=True), gemm_nt_split(sa, sb))
    with pytest.raises(RuntimeError):
        gemm_nt_split(sa, split_rows(b.to(gpu)))              # operands of different formats


@pytest.mark.parametrize("N,K", [(1, 1), (100, 37), (256, 64), (257, 300), (700, 1030)])
def test_gram_split2_is_symmetric(gpu, N, K):
    gen = torch.Generator(device="cpu").manual_seed(N + K)
    x = torch.randn(K, N, generator=gen)                       # the operand is x^T, read in place
    g = gram_split(split2_rows(x.to(gpu), transposed=True))
    want = x.double().numpy().T @ x.double().numpy()
    assert torch.equal(g, g.T)
    assert rel_max(g.cpu().numpy(), want) < 2.0 ** -19 + gemm_tol(K)
    acc = gram_split(split2_rows(x.to(gpu), transposed=True), out=g.clone(), alpha=1.0, beta=1.0)
    assert torch.equal(acc, acc.T) and rel_max(acc.cpu().numpy(), 2 * want) < 2.0 ** -19 + gemm_tol(K)


@pytest.mark.parametrize("M,N,K", [(1, 1, 1), (130, 70, 33), (256, 512, 64), (1000, 513, 257), (64, 2048, 4096), (129, 257, 8200)])
def test_gemm_nt_split(gpu, M, N, K):
    gen = torch.Generator(device="cpu").manual_seed(M * 7 + N + K)
    a, b = torch.randn(M, K, generator=gen), torch.randn(N, K, generator=gen)
    want = a.double().numpy() @ b.double().numpy().T
    got = gemm_nt_split(split_rows(a.to(gpu)), split_rows(b.to(gpu)))
    err = rel_max(got.cpu().numpy(), want)
    assert got.shape == (M, N) and err < gemm_tol(K)
    # no less accurate than the fp32 MFMA instruction on the same operands (factor 1.5 for noise)
    assert err <= 1.5 * rel_max(gemm_nt(a.to(gpu), b.to(gpu)).cpu().numpy(), want) + 1e-7
    # a transposed left operand, alpha, beta and the row scale epilogue
    at = a.T.contiguous()
    c0 = torch.randn(M, N, generator=gen)
    rs = torch.rand(M, generator=gen)
    got = gemm_nt_split(split_rows(at.to(gpu), transposed=True), split_rows(b.to(gpu)), out=c0.clone().to(gpu),
                        alpha=0.5, beta=-2.0, row_scale=rs.to(gpu))
    want2 = (0.5 * want - 2.0 * c0.double().numpy()) * rs.double().numpy()[:, None]
    assert rel_max(got.cpu().numpy(), want2) < gemm_tol(K)
    # strided output
    wide = torch.zeros(M, N + 5, device=gpu)
    gemm_nt_split(split_rows(a.to(gpu)), split_rows(b.to(gpu)), out=wide[:, 2 : 2 + N])
    assert rel_max(wide[:, 2 : 2 + N].cpu().numpy(), want) < gemm_tol(K)
    assert float(wide[:, :2].abs().sum()) == 0 and float(wide[:, 2 + N :].abs().sum()) == 0


@pytest.mark.parametrize("N,K", [(1, 1), (100, 37), (256, 64), (257, 300), (700, 1030)])
def test_gram_split_is_symmetric_and_accumulates(gpu, N, K):
    gen = torch.Generator(device="cpu").manual_seed(N + K)
    x = torch.randn(K, N, generator=gen)                      # the operand is x^T, as in X^T X
    want = x.double().numpy().T @ x.double().numpy()
    op = split_rows(x.to(gpu), transposed=True)
    got = gram_split(op)
    assert torch.equal(got, got.T)
    assert rel_max(got.cpu().numpy(), want) < gemm_tol(K)
    full = gemm_nt_split(op, op)
    if _lib.load().trakhip_gram_split_workspace(N, K, _lib.F32, 0) == 0:
        assert torch.equal(torch.tril(got), torch.tril(full))     # the same tiles, the same arithmetic
    else:                                                         # three shares of k, added in a fixed order
        assert rel_max(torch.tril(got).cpu().numpy(), torch.tril(full).cpu().numpy()) < gemm_tol(K)
    again = gram_split(op, out=got.clone(), alpha=0.5, beta=1.0)
    assert torch.equal(again, again.T)
    assert rel_max(again.cpu().numpy(), 1.5 * want) < gemm_tol(K)
    wide = torch.full((N, N + 3), 7.0, device=gpu)
    gram_split(op, out=wide[:, 1 : 1 + N])
    assert torch.equal(wide[:, 1 : 1 + N], got) and float((wide[:, 0] - 7).abs().sum()) == 0


def test_gemm_nt_split_keeps_small_terms(gpu):
    # b = 1 + 2^-20 needs 21 significand bits: one bf16 term (8 bits) would return exactly K, the
    # split product returns K * (1 + 2^-20) to fp32 accuracy (K small enough that the running sum
    # still resolves the small part, as for any fp32 dot product)
    K = 16
    a = torch.ones(32, K)
    b = torch.full((32, K), 1.0 + 2.0 ** -20)
    want = K * (1.0 + 2.0 ** -20)
    got = gemm_nt_split(split_rows(a.to(gpu)), split_rows(b.to(gpu))).cpu().numpy().astype(np.float64)
    assert np.abs(got - want).max() <= 2.0 ** -23 * K
    # cross terms of both operands: (1 + 2^-9)(1 - 2^-9) = 1 - 2^-18 needs a1*b2, a2*b1 and a2*b2
    a = torch.full((32, K), 1.0 + 2.0 ** -9)
    b = torch.full((32, K), 1.0 - 2.0 ** -9)
    got = gemm_nt_split(split_rows(a.to(gpu)), split_rows(b.to(gpu))).cpu().numpy().astype(np.float64)
    assert np.abs(got - K * (1.0 - 2.0 ** -18)).max() <= 2.0 ** -23 * K


@pytest.mark.parametrize("gemm", ["split", "split2", "fp32"])
@pytest.mark.parametrize("N,k,M,lam,max_dim", [(700, 512, 90, 1e-3, 20_000), (2500, 1024, 300, 0.0, 1000), (333, 100, 17, 1e-2, 100)])
def test_score_computer_matches_float64_oracle(gpu, N, k, M, lam, max_dim, gemm):
    gen = torch.Generator(device="cpu").manual_seed(N + k)
    X = torch.randn(N, k, generator=gen) / math.sqrt(k)
    Xt = torch.randn(M, k, generator=gen) / math.sqrt(k)
    otl = torch.rand(N, generator=gen)
    sc = BasicScoreComputer(dtype=torch.float32, device="cuda:0", CUDA_MAX_DIM_SIZE=max_dim, lambda_reg=lam, gemm=gemm)
    xtx_want = so.xtx_f64(X.numpy())
    feats_want, _, _ = so.x_xtx_inv_f64(X.numpy(), xtx_want, lam)
    scores_want = so.scores_f64(feats_want, Xt.numpy())

    for src in (X, X.to(gpu)):                               # host-resident (blocked) and device-resident
        xtx = sc.get_xtx(src)
        assert xtx.shape == (k, k) and rel_max(xtx.cpu().numpy(), xtx_want) < 1e-5
        feats = sc.get_x_xtx_inv(src, xtx)
        assert feats.shape == (N, k) and rel_max(feats.cpu().numpy(), feats_want) < 1e-4
        acc = torch.zeros(N, M)
        sc.get_scores(feats, Xt.to(gpu), accumulator=acc)     # [N_train, M_targets] (trak/score_computers.py:90)
        sc.get_scores(feats, Xt.to(gpu), accumulator=acc)
        assert rel_max(acc.numpy(), 2 * scores_want) < 1e-4
    # accumulator resident on the GPU: accumulated in the GEMM epilogue
    dev_acc = torch.zeros(N, M, device=gpu)
    sc.get_scores(feats, Xt.to(gpu), accumulator=dev_acc)
    sc.get_scores(feats, Xt.to(gpu), accumulator=dev_acc)
    assert rel_max(dev_acc.cpu().numpy(), 2 * scores_want) < 1e-4
    # fused finalize_scores epilogue (trak/traker.py:670-678) for one model
    fused = sc.get_scaled_scores(feats, Xt.to(gpu), otl.to(gpu))
    assert rel_max(fused.cpu().numpy(), so.finalize_scores_f64(scores_want, otl.numpy(), 1)) < 1e-4
    assert rel_max(get_matrix_mult(feats, Xt.to(gpu)).cpu().numpy(), scores_want) < 1e-4


@pytest.mark.parametrize("gemm", ["split", "split2", "fp32"])
def test_full_size_scoring_shape(gpu, gemm):
    """N = 50 000 training rows, k = 4096, M = 10 000 targets, lambda = 1e-3: the float64 oracle does not
    finish in seconds on a CPU at this size, so the check uses what does not depend on size: the
    inverse identity, the trace closed form, symmetry, and row / block samples of every product
    against float64 (1e-4 relative, the bar stated for the scores)."""
    N, k, M, lam = 50_000, 4096, 10_000, 1e-3
    gen = torch.Generator(device=gpu).manual_seed(20_011)
    X = torch.randn(N, k, generator=gen, device=gpu) / math.sqrt(k)
    Xt = torch.randn(M, k, generator=gen, device=gpu) / math.sqrt(k)
    otl = torch.rand(N, generator=gen, device=gpu)
    sc = BasicScoreComputer(dtype=torch.float32, device="cuda:0", lambda_reg=lam, gemm=gemm)
    xtx = sc.get_xtx(X)
    assert torch.equal(xtx, xtx.T)
    trace64 = float((X.double() ** 2).sum())
    # fp32 accumulation over 50 000 positive terms: the bound the GEMM tests use, not better
    assert abs(float(xtx.double().diagonal().sum()) - trace64) < gemm_tol(N) * trace64
    cols = torch.arange(1000, 1064, device=gpu)
    block64 = X[:, cols].double().T @ X.double()[:, 3000:3100]
    assert rel_max(xtx[cols][:, 3000:3100].cpu().numpy(), block64.cpu().numpy()) < gemm_tol(N)

    inv, mean_abs = spd_inverse(xtx, lambda_reg=lam, normalize=True)
    a64 = xtx.double() + lam * torch.eye(k, device=gpu, dtype=torch.float64)
    resid = a64 @ (inv.double() * mean_abs.double()) - torch.eye(k, device=gpu, dtype=torch.float64)
    assert float(resid.abs().max()) < 1e-4
    assert abs(float(inv.abs().mean()) - 1.0) < 1e-5                      # the rescaling of score_computers.py:166

    feats = sc.get_x_xtx_inv(X, xtx)
    rows = torch.tensor([0, 1, 777, 25_000, 49_999], device=gpu)
    inv64 = torch.linalg.inv(a64)
    inv64 = inv64 / inv64.abs().mean()
    feats64 = X[rows].double() @ inv64
    assert rel_max(feats[rows].cpu().numpy(), feats64.cpu().numpy()) < 1e-4

    acc = torch.zeros(N, M, device=gpu)
    sc.get_scores(feats, Xt, accumulator=acc)
    scores64 = feats64 @ Xt.double().T
    assert rel_max(acc[rows].cpu().numpy(), scores64.cpu().numpy()) < 1e-4
    tcols = torch.tensor([0, 5000, 9999], device=gpu)
    col64 = (X.double() @ inv64) @ Xt[tcols].double().T                    # every training row, three targets
    assert rel_max(acc[:, tcols].cpu().numpy(), col64.cpu().numpy()) < 1e-4
    fused = sc.get_scaled_scores(feats, Xt, otl)
    assert rel_max(fused[rows].cpu().numpy(), (scores64 * otl[rows].double()[:, None]).cpu().numpy()) < 1e-4


def test_score_computer_half_precision_flow(gpu):
    """TRAKer's default (use_half_precision): fp16 gradients and an fp16 score computer.  Every
    product runs from single fp16 planes (exact products); results are fp16 tensors as in the
    reference, compared with float64 computed from the same fp16 inputs at fp16 resolution."""
    N, k, M, lam = 900, 512, 70, 1e-2
    gen = torch.Generator(device="cpu").manual_seed(99)
    X = (torch.randn(N, k, generator=gen) / math.sqrt(k)).half()
    Xt = (torch.randn(M, k, generator=gen) / math.sqrt(k)).half()
    sc = BasicScoreComputer(dtype=torch.float16, device="cuda:0", lambda_reg=lam)
    xtx = sc.get_xtx(X.to(gpu))
    assert xtx.dtype == torch.float16
    x64 = X.double().numpy()
    assert rel_max(xtx.float().cpu().numpy(), x64.T @ x64) < 1e-3            # one fp16 rounding of the result
    feats = sc.get_x_xtx_inv(X.to(gpu), xtx)
    assert feats.dtype == torch.float16 and feats.shape == (N, k)
    inv64 = np.linalg.inv(xtx.double().cpu().numpy() + lam * np.eye(k))
    inv16 = torch.from_numpy(inv64 / np.abs(inv64).mean()).half().double().numpy()   # the reference casts the inverse
    assert rel_max(feats.float().cpu().numpy(), x64 @ inv16) < 3e-3
    acc = torch.zeros(N, M, device=gpu)
    sc.get_scores(feats, Xt.to(gpu), accumulator=acc)
    want = feats.double().cpu().numpy() @ Xt.double().numpy().T
    assert rel_max(acc.cpu().numpy(), want) < gemm_tol(k)                    # exact products, fp32 sums


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("where", ["cpu", "gpu"])
def test_blockwise_product_collects_on_the_host(gpu, dtype, where):
    """The host-collected block product (results too large for the device; trak/utils.py:135-245): ragged
    blocks in both directions, operands on either side, a CPU result of the target type, accumulation."""
    gen = torch.Generator(device="cpu").manual_seed(11)
    N, M, K = 300, 150, 128
    f, t = torch.randn(N, K, generator=gen).to(dtype), torch.randn(M, K, generator=gen).to(dtype)
    want = f.double().numpy() @ t.double().numpy().T
    src_f, src_t = (f, t) if where == "cpu" else (f.to(gpu), t.to(gpu))
    tol = gemm_tol(K) if dtype == torch.float32 else 1e-3                      # the result is rounded to fp16
    got = utils_module.get_matrix_mult_blockwise(src_f, src_t, dtype, bs=64, block_bytes=64 * 64 * 4)
    assert got.device.type == "cpu" and got.dtype == dtype and got.shape == (N, M)
    assert rel_max(got.numpy(), want) < tol
    # the same through the public entry point, and one block when it fits
    assert torch.equal(get_matrix_mult(src_f, src_t, use_blockwise=True, batch_size=8096), utils_module.get_matrix_mult_blockwise(src_f, src_t))
    acc = torch.ones(N, M)
    utils_module.get_matrix_mult_blockwise(src_f, src_t, out=acc, accumulate=True, bs=64, block_bytes=64 * 64 * 4)
    utils_module.get_matrix_mult_blockwise(src_f, src_t, out=acc, accumulate=True, bs=100, block_bytes=100 * 100 * 4)
    assert rel_max(acc.numpy(), 1.0 + 2.0 * want) < tol + 1e-6


def test_get_scores_goes_blockwise_when_the_result_does_not_fit(gpu, monkeypatch):
    gen = torch.Generator(device="cpu").manual_seed(12)
    N, M, k = 500, 70, 256
    feats, Xt = torch.randn(N, k, generator=gen) / 16, torch.randn(M, k, generator=gen) / 16
    want = feats.double().numpy() @ Xt.double().numpy().T
    calls = []
    real = utils_module.get_matrix_mult_blockwise

    def spy(*args, **kwargs):
        calls.append(1)
        return real(*args, bs=64, block_bytes=128 * 64 * 4, **kwargs)

    monkeypatch.setattr(score_computers_module, "output_fits_on_device", lambda *a, **k: False)
    monkeypatch.setattr(score_computers_module, "get_matrix_mult_blockwise", spy)
    for gemm in ("split", "split2", "fp32"):
        sc = BasicScoreComputer(dtype=torch.float32, device="cuda:0", gemm=gemm)
        acc = torch.zeros(N, M)
        sc.get_scores(feats.to(gpu), Xt.to(gpu), accumulator=acc)
        sc.get_scores(feats, Xt, accumulator=acc)                                 # host-resident operands
        assert rel_max(acc.numpy(), 2 * want) < 1e-5
    assert len(calls) == 6
    # a device accumulator never takes this path
    dev_acc = torch.zeros(N, M, device=gpu)
    BasicScoreComputer(dtype=torch.float32, device="cuda:0").get_scores(feats.to(gpu), Xt.to(gpu), accumulator=dev_acc)
    assert len(calls) == 6 and rel_max(dev_acc.cpu().numpy(), want) < 1e-5


@pytest.mark.parametrize("fmt", ["fp32", "two_planes", "fp16", "bf16"])
@pytest.mark.parametrize("N,K", [(300, 5000), (1000, 3100), (4096, 2048)])
def test_gram_shares_the_k_range_over_idle_cus(gpu, fmt, N, K):
    """A symmetric product with few tiles and a long k range runs as three shares that are added in a
    fixed order: same accuracy as the one-piece product, exactly symmetric, repeatable bit for bit,
    accumulation into an earlier result."""
    gen = torch.Generator(device=gpu).manual_seed(N + K)
    x = torch.randn(K, N, generator=gen, device=gpu)            # the operand is x^T, read in place
    if fmt in ("fp16", "bf16"):
        x = x.to(torch.float16 if fmt == "fp16" else torch.bfloat16)
    make = (lambda: split2_rows(x, transposed=True)) if fmt == "two_planes" else (lambda: split_rows(x, transposed=True))
    g = gram_split(make())
    want = (x.double().T @ x.double()).cpu().numpy()
    tol = (2.0 ** -19 if fmt == "two_planes" else 0.0) + gemm_tol(K)
    assert torch.equal(g, g.T) and rel_max(g.cpu().numpy(), want) < tol
    assert torch.equal(g, gram_split(make()))
    acc = gram_split(make(), out=g.clone(), alpha=0.5, beta=2.0)
    assert torch.equal(acc, acc.T) and rel_max(acc.cpu().numpy(), 2.5 * want) < tol
    # a padded destination keeps its padding
    wide = torch.full((N, N + 3), 7.0, device=gpu)
    gram_split(make(), out=wide[:, :N])
    assert torch.equal(wide[:, :N], g) and bool((wide[:, N:] == 7.0).all())
