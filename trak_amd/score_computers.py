"""Score computer plug-in with the interface of the reference's trak/score_computers.py,
running the three GEMMs and the regularized inverse on the GPU through libtrakhip.

`TRAKer(score_computer=BasicScoreComputer)` constructs it as
`cls(dtype=, device=, logging_level=, lambda_reg=)` (trak/traker.py:186-193) and calls
`get_xtx`, `get_x_xtx_inv` and `get_scores` (trak/traker.py:483-485, :667).
"""
import logging
from abc import ABC, abstractmethod

import torch
from torch import Tensor

from .utils import gemm_nt, gemm_tn, spd_inverse

ch = torch


class AbstractScoreComputer(ABC):
    """Interface of trak/score_computers.py:22-91."""

    @abstractmethod
    def __init__(self, dtype, device) -> None:
        self.dtype = dtype
        self.device = device

    @abstractmethod
    def get_xtx(self, grads: Tensor) -> Tensor:
        """X^T X for projected gradients X of shape (n, p)."""

    @abstractmethod
    def get_x_xtx_inv(self, grads: Tensor, xtx: Tensor) -> Tensor:
        """X (X^T X)^-1 of shape (n, p)."""

    @abstractmethod
    def get_scores(self, features: Tensor, target_grads: Tensor, accumulator: Tensor) -> None:
        """accumulator (n, m) += features (n, p) @ target_grads (m, p)^T."""


class BasicScoreComputer(AbstractScoreComputer):
    """GPU implementation of the reference's BasicScoreComputer (trak/score_computers.py:119-189).

    All arithmetic is fp32 on the device (fp32 MFMA); `dtype` is the type of the returned
    tensors, as in the reference.  Inputs may live on the host: they are moved block by block
    (CUDA_MAX_DIM_SIZE rows at a time), which is what the reference's `block.to(self.device)`
    does.
    """

    def __init__(
        self,
        dtype: torch.dtype,
        device,
        CUDA_MAX_DIM_SIZE: int = 20_000,
        logging_level=logging.INFO,
        lambda_reg: float = 0.0,
    ) -> None:
        super().__init__(dtype, device)
        self.CUDA_MAX_DIM_SIZE = CUDA_MAX_DIM_SIZE
        self.logger = logging.getLogger("ScoreComputer")
        self.logger.setLevel(logging_level)
        self.lambda_reg = lambda_reg
        dev = ch.device(device)
        if dev.type != "cuda":
            raise ValueError("BasicScoreComputer of trak_amd computes on a GPU; pass a cuda device")
        self._dev = dev

    def _blocks(self, grads):
        if grads.device == self._dev or (grads.is_cuda and self._dev.index is None):
            return [grads]  # resident: one pass, the kernel walks all rows
        return ch.split(grads, split_size_or_sections=self.CUDA_MAX_DIM_SIZE, dim=0)

    def get_xtx(self, grads: Tensor) -> Tensor:
        self.proj_dim = grads.shape[1]
        result = ch.zeros(self.proj_dim, self.proj_dim, dtype=ch.float32, device=self._dev)
        for block in self._blocks(grads):
            block = block.to(self._dev)
            gemm_tn(block, block, out=result, alpha=1.0, beta=1.0)
        return result.to(self.dtype)

    def get_x_xtx_inv(self, grads: Tensor, xtx: Tensor) -> Tensor:
        # (xtx + lambda I)^-1 in fp32, divided by the mean absolute entry
        # (trak/score_computers.py:160-166)
        xtx_inv, _ = spd_inverse(xtx.to(self._dev), lambda_reg=self.lambda_reg, normalize=True)
        xtx_inv = xtx_inv.to(self.dtype)

        result = ch.empty(grads.shape[0], xtx_inv.shape[1], dtype=ch.float32, device=self._dev)
        start = 0
        for block in self._blocks(grads):
            end = start + block.shape[0]
            # the inverse is symmetric, so block @ inv == block @ inv^T
            gemm_nt(block.to(self._dev), xtx_inv, out=result[start:end])
            start = end
        return result.to(self.dtype)

    def get_scores(self, features: Tensor, target_grads: Tensor, accumulator: Tensor) -> None:
        train_dim = features.shape[0]
        target_dim = target_grads.shape[0]
        self.logger.debug(f"{train_dim=}, {target_dim=}")
        f, t = features.to(self._dev), target_grads.to(self._dev)
        if (
            accumulator.is_cuda
            and accumulator.device == f.device
            and accumulator.dtype == ch.float32
            and accumulator.dim() == 2
            and accumulator.stride(1) == 1
        ):
            # accumulator on the GPU: the sum over checkpoints happens in the GEMM epilogue and the
            # [N, M] matrix never crosses PCIe per checkpoint (trak/traker.py:641-668 moves it each time)
            gemm_nt(f, t, out=accumulator, alpha=1.0, beta=1.0)
            return
        scores = gemm_nt(f, t)
        if accumulator.is_cuda:
            accumulator += scores.to(accumulator.dtype)
        else:
            accumulator += scores.to(accumulator.dtype).detach().cpu()

    def get_scaled_scores(self, features: Tensor, target_grads: Tensor, out_to_loss: Tensor, scale: float = 1.0):
        """scale * (features @ target_grads^T) with row i multiplied by out_to_loss[i], on the
        device: the finalize_scores epilogue of trak/traker.py:670-678 fused into the GEMM."""
        return gemm_nt(
            features.to(self._dev), target_grads.to(self._dev), alpha=scale, row_scale=out_to_loss.reshape(-1)
        )
