"""Pins the CPU baselines (restatements of BasicProjector and BasicScoreComputer) with closed
forms and textbook identities."""
import math

import numpy as np
import torch

from oracle import score_oracle as so
from oracle.basic_projector import BasicProjectorCPU


def test_basic_projector_block_seeds_and_shapes():
    p = BasicProjectorCPU(grad_dim=1000, proj_dim=512, seed=42, proj_type="rademacher")
    assert p.block_size == 100 and p.num_blocks == 6          # trak/projectors.py:240-241
    assert p.block_seeds(0) == [42, 1042, 2042, 3042, 4042, 5042]
    assert p.block_seeds(3)[0] == 42 + 300000                  # :262-264
    q = BasicProjectorCPU(grad_dim=10, proj_dim=20, seed=0, proj_type="normal")
    assert q.block_size == 20 and q.num_blocks == 1


def test_basic_projector_matrix_and_jl_property():
    torch.manual_seed(0)
    P, k = 20_000, 512
    p = BasicProjectorCPU(grad_dim=P, proj_dim=k, seed=7, proj_type="rademacher")
    m = p.generate_block(7).clone()
    assert set(m.unique().tolist()) == {-1.0, 1.0} and abs(m.mean().item()) < 5 / math.sqrt(m.numel())
    assert torch.equal(p.generate_block(7), m)               # same seed, same block
    g = torch.randn(4, P)
    out = p.project(g, model_id=0)
    assert out.shape == (4, k)
    # block 0 of the sketch is grads @ block matrix of seed 7
    assert torch.allclose(out[:, :100], g @ m, atol=1e-3)
    ratio = out.norm(dim=1) / (g.norm(dim=1) * math.sqrt(k))
    assert torch.all((ratio - 1).abs() < 5 / math.sqrt(2 * k) + 0.05)
    out2 = p.project(g, model_id=1)
    assert not torch.allclose(out, out2)
    n = BasicProjectorCPU(grad_dim=P, proj_dim=100, seed=1, proj_type="normal").generate_block(1)
    assert abs(n.mean().item()) < 5 / math.sqrt(n.numel()) and abs(n.var().item() - 1) < 0.01


def test_score_oracle_identities():
    rng = np.random.default_rng(0)
    N, k, M = 300, 24, 17
    X = rng.standard_normal((N, k))
    xtx = so.xtx_f64(X)
    assert np.allclose(xtx, xtx.T) and np.allclose(xtx, sum(np.outer(r, r) for r in X))
    lam = 0.3
    feats, inv, mean_abs = so.x_xtx_inv_f64(X, xtx, lam)
    assert np.allclose((xtx + lam * np.eye(k)) @ inv, np.eye(k), atol=1e-10)
    assert np.isclose(np.abs(inv / mean_abs).mean(), 1.0)
    assert np.allclose(feats * mean_abs, X @ inv)
    # lambda = 0: features^T X * mean_abs = I
    f0, _, m0 = so.x_xtx_inv_f64(X, xtx, 0.0)
    assert np.allclose(f0.T @ X * m0, np.eye(k), atol=1e-9)
    # orthonormal columns: XtX = I, inverse = I / (1 + lambda)
    Q, _ = np.linalg.qr(rng.standard_normal((N, k)))
    assert np.allclose(so.xtx_f64(Q), np.eye(k), atol=1e-12)
    _, invq, _ = so.x_xtx_inv_f64(Q, so.xtx_f64(Q), 1.0)
    assert np.allclose(invq, np.eye(k) / 2.0, atol=1e-12)
    # diagonal X
    d = np.arange(1, k + 1, dtype=np.float64)
    _, invd, _ = so.x_xtx_inv_f64(np.diag(d), np.diag(d**2), 0.5)
    assert np.allclose(np.diag(invd), 1.0 / (d**2 + 0.5))
    Xt = rng.standard_normal((M, k))
    S = so.scores_f64(feats, Xt)
    assert S.shape == (N, M) and np.isclose(S[3, 5], feats[3] @ Xt[5])
    otl = rng.uniform(size=N)
    fin = so.finalize_scores_f64(2 * S, 2 * otl, 2)
    assert np.allclose(fin, S * otl[:, None])


def test_cpu_score_computer_matches_f64_and_is_block_independent():
    torch.manual_seed(1)
    N, k, M = 257, 32, 9
    X = torch.randn(N, k) / math.sqrt(k)
    Xt = torch.randn(M, k) / math.sqrt(k)
    a = so.BasicScoreComputerCPU(lambda_reg=1e-3, max_dim=100)   # 3 ragged blocks
    b = so.BasicScoreComputerCPU(lambda_reg=1e-3, max_dim=20_000)
    xa, xb = a.get_xtx(X), b.get_xtx(X)
    assert torch.allclose(xa, xb, atol=1e-5)
    fa, fb = a.get_x_xtx_inv(X, xa), b.get_x_xtx_inv(X, xb)
    assert torch.allclose(fa, fb, rtol=1e-4, atol=1e-5)
    acc = torch.zeros(N, M)
    a.get_scores(fa, Xt, acc)
    a.get_scores(fa, Xt, acc)
    f64, _, _ = so.x_xtx_inv_f64(X.numpy(), so.xtx_f64(X.numpy()), 1e-3)
    want = 2 * so.scores_f64(f64, Xt.numpy())
    assert np.abs(acc.numpy() - want).max() / np.abs(want).max() < 1e-4
