"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's BasicScoreComputer
(trak/score_computers.py:119-189, trak/utils.py:128-132) and of the score epilogue of
TRAKer.finalize_scores (trak/traker.py:670-678).

Two forms:
  * `*_f64`: numpy float64, the parity oracle for the GPU kernels;
  * `BasicScoreComputerCPU`: torch CPU float32 with the reference's blocking, the
    `cpu_baseline` bench.py times.
Pinned by textbook identities (tests/test_oracle_baselines.py): (XtX + lambda I) inv = I,
orthonormal columns give XtX = I, diagonal closed form, block-split independence, and
agreement between the two forms.
"""
import numpy as np
import torch

CUDA_MAX_DIM_SIZE = 20_000  # trak/score_computers.py:127


def xtx_f64(X):
    X = np.asarray(X, dtype=np.float64)
    return X.T @ X  # trak/score_computers.py:145-155


def x_xtx_inv_f64(X, xtx, lambda_reg):
    """features = X @ (inv / mean|inv|), inv = (xtx + lambda I)^-1 (trak/score_computers.py:157-177).
    Returns (features, inverse before the rescale, mean|inv|)."""
    X = np.asarray(X, dtype=np.float64)
    xtx = np.asarray(xtx, dtype=np.float64)
    inv = np.linalg.inv(xtx + lambda_reg * np.eye(xtx.shape[0]))
    mean_abs = np.abs(inv).mean()
    return X @ (inv / mean_abs), inv, mean_abs


def scores_f64(features, target_grads):
    """[N_train, M_targets] = features @ target_grads^T (trak/utils.py:131, orientation of
    trak/score_computers.py:90)."""
    return np.asarray(features, dtype=np.float64) @ np.asarray(target_grads, dtype=np.float64).T


def finalize_scores_f64(acc, out_to_loss_sum, num_models):
    """scores = (acc / num_models) * (sum of out_to_loss / num_models), out_to_loss [N, 1]
    broadcast over targets (trak/traker.py:670-678)."""
    acc = np.asarray(acc, dtype=np.float64)
    otl = np.asarray(out_to_loss_sum, dtype=np.float64).reshape(-1, 1)
    return (acc / num_models) * (otl / num_models)


class BasicScoreComputerCPU:
    """torch-CPU float32 restatement with the reference's row blocking."""

    def __init__(self, dtype=torch.float32, lambda_reg=0.0, max_dim=CUDA_MAX_DIM_SIZE):
        self.dtype = dtype
        self.lambda_reg = lambda_reg
        self.max_dim = max_dim

    def get_xtx(self, grads):
        k = grads.shape[1]
        result = torch.zeros(k, k, dtype=self.dtype)
        for block in torch.split(grads, self.max_dim, dim=0):
            result += block.T @ block
        return result

    def get_x_xtx_inv(self, grads, xtx):
        xtx_reg = xtx + self.lambda_reg * torch.eye(xtx.size(0), dtype=xtx.dtype)
        xtx_inv = torch.linalg.inv(xtx_reg.to(torch.float32))
        xtx_inv /= xtx_inv.abs().mean()
        xtx_inv = xtx_inv.to(self.dtype)
        result = torch.empty(grads.shape[0], xtx_inv.shape[1], dtype=self.dtype)
        for i, block in enumerate(torch.split(grads, self.max_dim, dim=0)):
            start = i * self.max_dim
            end = min(grads.shape[0], (i + 1) * self.max_dim)
            result[start:end] = block @ xtx_inv
        return result

    def get_scores(self, features, target_grads, accumulator):
        accumulator += (features @ target_grads.t()).clone().to(features.dtype)
