"""Bounded randomized parity tests (fixed seeds, a time budget, the first mismatch fails the test).

Projection: random (rows, features, proj_dim, feature tiles, element type, matrix type, dense matrix or list of
tensors) through the C ABI against the CPU oracle's float64 contraction on a window of columns, the list
form against the dense form bit for bit.  GEMMs: random (M, N, K, alpha, beta, element type, kernel family)
against float64.  The inverse of matrices that are not positive definite: random sizes and structures against
the float64 inverse, with a bound that follows the condition number.  The fixed-shape tests cover the cases somebody thought of; these cover combinations nobody
listed.
"""
import math
import random
import time

import numpy as np
import pytest
import torch

from oracle import jl_oracle as npo
from trak_amd import fast_jl
from trak_amd.utils import (gemm_nt, gemm_nt16, gemm_nt_split, gemm_tn, general_inverse, gram_split, split2_rows,
                            split_rows)

pytestmark = pytest.mark.gpu

TOL = {torch.float16: 1e-3, torch.bfloat16: 1e-3, torch.float32: 1e-5}
NAMES = {npo.RADEMACHER: "rademacher", npo.NORMAL: "normal"}
BUDGET_S = 25.0   # per test; the case lists below finish well inside it on an MI355X box


def _rel_rows(got, want):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    return float((np.linalg.norm(got - want, axis=1) / np.maximum(np.linalg.norm(want, axis=1), 1e-300)).max())


def test_random_projection_shapes_against_the_oracle(gpu, c_oracle):
    rng = random.Random(20_261)
    gen = torch.Generator(device="cpu").manual_seed(20_262)
    t0 = time.monotonic()
    done = 0
    for it in range(60):
        if time.monotonic() - t0 > BUDGET_S:
            break
        B = rng.choice([1, 2, 7, 16, 31, 32, 33, 40, 63, 64, 65, 97, 130])
        P = rng.choice([1, 3, 25, 255, 256, 257, 511, 1000, 4097, 9001, 20_000, 33_333, 65_537, 100_003, 262_144])
        k = rng.choice([512, 1024, 1536, 2048, 2560, 3072, 5120])
        tiles = rng.choice([1, 2, 7, 64, 108, 256, 304])
        dt = rng.choice([torch.float16, torch.bfloat16, torch.float32])
        pt = rng.choice([npo.RADEMACHER, npo.NORMAL])
        seed = rng.randrange(0, 2**32)
        case = (it, B, P, k, tiles, dt, NAMES[pt], seed)
        g = (torch.randn(B, P, generator=gen) * 10 ** rng.uniform(-4, 0)).to(dt).to(gpu)
        out = getattr(fast_jl, f"project_{NAMES[pt]}_32")(g, k, seed, tiles)
        assert out.shape == (B, k) and out.dtype == torch.float32, case
        c0 = rng.choice([0, 480, k - 32, k // 2 - 16, 1024 - 32 if k >= 1024 else 0])
        want = c_oracle.project(g.float().cpu().numpy(), seed, tiles, c0, 32, pt)
        err = _rel_rows(out[:, c0:c0 + 32].cpu().numpy(), want)
        assert err < TOL[dt], (case, c0, err)
        # the same gradient as a list of tensors cut at random features: the same bits
        cuts = sorted(set([0, P] + [rng.randrange(0, P + 1) for _ in range(rng.choice([0, 1, 3, 6]))]))
        pieces = [g[:, a:b].contiguous() if rng.random() < 0.5 else g[:, a:b] for a, b in zip(cuts[:-1], cuts[1:]) if b > a]
        gathered = fast_jl.project_gather(pieces, k, seed, tiles, NAMES[pt])
        assert torch.equal(gathered, out), case
        done += 1
    assert done >= 15, done   # the budget must not silently turn the test into nothing


def _tol(K):
    return 1e-6 + 2e-7 * math.sqrt(K)


def _rel(got, want):
    want = np.asarray(want, np.float64)
    return float(np.abs(np.asarray(got, np.float64) - want).max() / max(np.abs(want).max(), 1e-300))


def test_random_gemm_shapes_against_float64(gpu):
    rng = random.Random(1234)
    gen = torch.Generator(device="cpu").manual_seed(7)
    t0 = time.monotonic()
    done = 0
    for it in range(60):
        if time.monotonic() - t0 > BUDGET_S:
            break
        M = rng.choice([1, 5, 31, 64, 127, 128, 129, 255, 256, 257, 300, 511, 700, 1025])
        N = rng.choice([1, 7, 32, 100, 128, 130, 256, 258, 513, 640])
        K = rng.choice([1, 8, 16, 40, 64, 96, 120, 128, 129, 192, 256, 1000, 2048])
        alpha, beta = rng.choice([1.0, 2.0]), rng.choice([0.0, 1.0, -0.5])
        case = (it, M, N, K, alpha, beta)
        a, b, c0 = torch.randn(M, K, generator=gen), torch.randn(N, K, generator=gen), torch.randn(M, N, generator=gen)
        a64, b64, c64 = a.double().numpy(), b.double().numpy(), c0.double().numpy()
        want = alpha * (a64 @ b64.T) + beta * c64
        ad, bd = a.to(gpu), b.to(gpu)
        got = gemm_nt(ad, bd, out=c0.clone().to(gpu), alpha=alpha, beta=beta)
        assert _rel(got.cpu().numpy(), want) < 2 * _tol(K), ("fp32 MFMA", case)
        got = gemm_nt_split(split_rows(ad), split_rows(bd), out=c0.clone().to(gpu), alpha=alpha, beta=beta)
        assert _rel(got.cpu().numpy(), want) < 2 * _tol(K), ("three bf16 planes", case)
        got = gemm_nt_split(split2_rows(ad), split2_rows(bd), out=c0.clone().to(gpu), alpha=alpha, beta=beta)
        bound = alpha * (np.abs(a64) @ np.abs(b64).T) + abs(beta) * np.abs(c64)
        assert np.all(np.abs(got.cpu().double().numpy() - want) <= bound * (2.0 ** -20 + 2e-7 * math.sqrt(K)) + 1e-30), \
            ("two fp16 planes", case)
        # A^T B through the TN kernel (the X^T X product)
        at = a.T.contiguous().to(gpu)                       # [K, M]
        bt = b.T.contiguous().to(gpu)                       # [K, N]
        got = gemm_tn(at, bt, out=c0.clone().to(gpu), alpha=alpha, beta=beta)
        assert _rel(got.cpu().numpy(), want) < 2 * _tol(K), ("fp32 MFMA TN", case)
        if K % 64 == 0:
            for dt in (torch.float16, torch.bfloat16):
                ah, bh = a.to(dt).to(gpu), b.to(dt).to(gpu)
                w = alpha * (ah.double().cpu().numpy() @ bh.double().cpu().numpy().T) + beta * c64
                got = gemm_nt16(ah, bh, out=c0.clone().to(gpu), alpha=alpha, beta=beta)
                assert _rel(got.cpu().numpy(), w) < 2 * _tol(K), ("16-bit in place", dt, case)
        done += 1
    assert done >= 15, done


def test_random_gram_shapes_against_float64(gpu):
    rng = random.Random(99)
    gen = torch.Generator(device="cpu").manual_seed(9)
    for N, K in [(1, 5000), (255, 3000), (513, 9000), (2049, 2000), (rng.choice([700, 1300, 1800]), rng.choice([640, 1536, 4100]))]:
        x = torch.randn(K, N, generator=gen)
        for kind, make in (("three bf16 planes", lambda t: split_rows(t, transposed=True)),
                           ("two fp16 planes", lambda t: split2_rows(t, transposed=True)),
                           ("one fp16 plane", lambda t: split_rows(t.half(), transposed=True))):
            op = make(x.to(gpu))
            got = gram_split(op)
            src = x.half().double() if op.dtype == torch.float16 else x.double()
            want = (src.T @ src).numpy()
            assert torch.equal(got, got.T), (kind, N, K)
            assert _rel(got.cpu().numpy(), want) < 2.0 ** -19 + _tol(K), (kind, N, K)


def test_random_matrices_through_the_general_inverse(gpu):
    # sizes on both sides of the routes' limits are covered by fixed tests; here the structure varies: what the
    # pivoting meets (rows of very different size, near-permutations, low rank + noise, symmetric indefinite)
    rng = random.Random(4711)
    gen = torch.Generator(device="cpu").manual_seed(4712)
    for it in range(14):
        n = rng.choice([3, 17, 64, 129, 200, 333, 512, 777, 1000, 1290])
        kind = rng.choice(["normal", "graded_rows", "near_permutation", "low_rank_noise", "symmetric_indefinite"])
        if kind == "normal":
            a = torch.randn(n, n, generator=gen)
        elif kind == "graded_rows":
            a = torch.randn(n, n, generator=gen) * 10 ** (-3 * torch.rand(n, 1, generator=gen))
        elif kind == "near_permutation":
            a = 1e-3 * torch.randn(n, n, generator=gen)
            a[torch.arange(n), torch.randperm(n, generator=gen)] += 1 + torch.rand(n, generator=gen)
        elif kind == "low_rank_noise":
            u = torch.randn(n, max(1, n // 20), generator=gen)
            a = u @ u.T / u.shape[1] + 1e-2 * torch.randn(n, n, generator=gen)
        else:
            x = torch.randn(n, n, generator=gen) / math.sqrt(n)
            a = (x + x.T) / 2 + torch.diag(torch.where(torch.rand(n, generator=gen) < 0.5, -1.0, 1.0))
        lam = rng.choice([0.0, 1e-3])
        case = (it, n, kind, lam)
        got, mean_abs = general_inverse(a.to(gpu), lambda_reg=lam)
        a64 = a.double().numpy() + lam * np.eye(n)
        want = np.linalg.inv(a64)
        cond = np.linalg.norm(a64, 1) * np.linalg.norm(want, 1)
        err = np.abs(got.cpu().numpy() - want).max() / np.abs(want).max()
        # LU with partial pivoting in fp32 measures 0.02 .. 0.05 of cond * 2^-24 on such matrices
        assert err <= 0.5 * cond * 2.0 ** -24 + 1e-6, (case, err, cond)
        assert abs(mean_abs.item() - np.abs(want).mean()) <= (0.5 * cond * 2.0 ** -24 + 1e-5) * np.abs(want).max(), case
