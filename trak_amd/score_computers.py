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

from .utils import (
    gemm_nt,
    gemm_nt16,
    gemm_nt_split,
    gemm_tn,
    get_matrix_mult_blockwise,
    gram_split,
    matmul_nt,
    nt16_ok,
    output_fits_on_device,
    scores_finalize,
    spd_inverse,
    split2_rows,
    split_rows,
)

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

    All arithmetic has fp32 accuracy on the device; `dtype` is the type of the returned tensors,
    as in the reference.  Inputs may live on the host: they are moved block by block
    (CUDA_MAX_DIM_SIZE rows at a time), which is what the reference's `block.to(self.device)`
    does.

    `gemm` selects how the three matrix products are computed: "split" (default) splits every
    fp32 operand exactly into three bf16 terms and runs six bf16 MFMAs per k step with fp32
    accumulation (same error as the fp32 instruction, 1.7 times its speed); "fp32" uses the fp32
    MFMA instruction directly; "split2" is an opt-in cheaper split for fp32 operands (rows scaled by a
    power of two, two fp16 planes, three MFMAs per k step: entries keep 22 significand bits relative
    to their row's largest magnitude instead of all 24; 1.75 times the speed of "split").  fp16 / bf16
    operands are multiplied as they are (exact products) under "split" and "split2".

    Differences from the reference that a caller can meet:
      * the device must be a GPU (the reference also runs on "cpu");
      * `X^T X + lambda I` is inverted by a Cholesky factorization.  When that fails - the matrix is
        symmetric but not positive definite, which happens to a Gram matrix that was rounded to fp16
        (TRAKer's default) or has deficient rank (fewer training points than proj_dim with
        lambda_reg = 0) - the matrix is inverted by this library's elimination with partial pivoting
        (`utils.general_inverse`: the pivoting of the LU behind the reference's torch.linalg.inv,
        trak/score_computers.py:163; matrices up to 12288 x 12288) and a warning is logged; an exactly
        singular matrix (a zero pivot) raises torch.linalg.LinAlgError as the reference's call does, an
        inverse with huge or non-finite entries is handed on as it is;
      * sums are kept in fp32 and rounded to `dtype` once.  accumulate_in_dtype=True reproduces the
        reference's arithmetic instead: `X^T X` is the sum over blocks of CUDA_MAX_DIM_SIZE rows of
        block products each rounded to `dtype`, the running sum rounded to `dtype` after every
        block (trak/score_computers.py:147-153), and lambda is added in the dtype of `xtx`
        (:160-162).  It costs one pass per block and only matters for fp16 / bf16 `dtype`.
    """

    def __init__(
        self,
        dtype: torch.dtype,
        device,
        CUDA_MAX_DIM_SIZE: int = 20_000,
        logging_level=logging.INFO,
        lambda_reg: float = 0.0,
        gemm: str = "split",
        accumulate_in_dtype: bool = False,
    ) -> None:
        super().__init__(dtype, device)
        self.accumulate_in_dtype = accumulate_in_dtype
        if gemm not in ("split", "split2", "fp32"):
            raise ValueError('gemm must be "split", "split2" or "fp32"')
        self.gemm = gemm
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

    def _gram(self, block, out, beta):
        if self.gemm != "fp32":
            # the operand is block^T, read in place; lower-triangle tiles + mirror image
            gram_split(self._split(block, transposed=True), out=out, alpha=1.0, beta=beta)
        else:
            gemm_tn(block, block, out=out, alpha=1.0, beta=beta)

    def get_xtx(self, grads: Tensor) -> Tensor:
        self.proj_dim = grads.shape[1]
        if self.accumulate_in_dtype:
            # trak/score_computers.py:147-153 to the letter: `result += block.T @ block` with both sides
            # in `dtype`, blocks of CUDA_MAX_DIM_SIZE rows wherever the gradients live
            result = ch.zeros(self.proj_dim, self.proj_dim, dtype=self.dtype, device=self._dev)
            product = ch.empty(self.proj_dim, self.proj_dim, dtype=ch.float32, device=self._dev)
            for block in ch.split(grads, split_size_or_sections=self.CUDA_MAX_DIM_SIZE, dim=0):
                self._gram(block.to(self._dev), product, 0.0)
                result += product.to(block.dtype)  # the block product in the gradients' type, as `block.T @ block` returns it
            return result
        result = ch.zeros(self.proj_dim, self.proj_dim, dtype=ch.float32, device=self._dev)
        for block in self._blocks(grads):
            self._gram(block.to(self._dev), result, 1.0)
        return result.to(self.dtype)

    def get_x_xtx_inv(self, grads: Tensor, xtx: Tensor) -> Tensor:
        # (xtx + lambda I)^-1 in fp32, divided by the mean absolute entry
        # (trak/score_computers.py:160-166)
        xtx = xtx.to(self._dev)
        if self.accumulate_in_dtype:
            # lambda is added in the dtype of xtx (trak/score_computers.py:160-162), then fp32
            xtx_reg = xtx + self.lambda_reg * ch.eye(xtx.size(dim=0), device=xtx.device, dtype=xtx.dtype)
            xtx_inv, _ = spd_inverse(xtx_reg, lambda_reg=0.0, normalize=True, general_fallback=True)
        else:
            xtx_inv, _ = spd_inverse(xtx, lambda_reg=self.lambda_reg, normalize=True, general_fallback=True)
        xtx_inv = xtx_inv.to(self.dtype)

        result = ch.empty(grads.shape[0], xtx_inv.shape[1], dtype=ch.float32, device=self._dev)
        # 16-bit gradients meet the inverse cast to their type (as in the reference) as single planes
        half = grads.dtype == xtx_inv.dtype and grads.dtype in (ch.float16, ch.bfloat16)
        inv_split = None  # planes of the inverse, made when the first block needs them
        start = 0
        for block in self._blocks(grads):
            end = start + block.shape[0]
            # the inverse is symmetric, so block @ inv == block @ inv^T
            if self.gemm != "fp32":
                block = block.to(self._dev)
                if half and nt16_ok(block, xtx_inv):
                    gemm_nt16(block, xtx_inv, out=result[start:end])
                else:
                    if inv_split is None:
                        inv_split = self._split(xtx_inv if half else xtx_inv.float())
                    gemm_nt_split(self._split(block if half else block.float()), inv_split, out=result[start:end])
            else:
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
            self._matmul_nt(f, t, out=accumulator, beta=1.0)
            return
        if not accumulator.is_cuda and not output_fits_on_device(train_dim, target_dim, self._dev):
            # too large for the device: block by block into the host accumulator (trak/utils.py:135-245)
            get_matrix_mult_blockwise(f, t, out=accumulator, accumulate=True,
                                      product=lambda a, b, o: self._matmul_nt(a, b, out=o))
            return
        scores = self._matmul_nt(f, t)
        if accumulator.is_cuda:
            accumulator += scores.to(accumulator.dtype)
        else:
            accumulator += scores.to(accumulator.dtype).detach().cpu()

    def get_scaled_scores(self, features: Tensor, target_grads: Tensor, out_to_loss: Tensor, scale: float = 1.0):
        """scale * (features @ target_grads^T) with row i multiplied by out_to_loss[i], on the
        device: the finalize_scores epilogue of trak/traker.py:670-678 fused into the GEMM."""
        return self._matmul_nt(
            features.to(self._dev), target_grads.to(self._dev), alpha=scale, row_scale=out_to_loss.reshape(-1)
        )

    def _split(self, t, transposed=False):
        """Operand format of the chosen product: 16-bit matrices stay one plane; fp32 ones become three
        exact bf16 planes ("split") or two scaled fp16 planes ("split2")."""
        if self.gemm == "split2" and t.dtype not in (ch.float16, ch.bfloat16):
            return split2_rows(t, transposed=transposed)
        return split_rows(t, transposed=transposed)

    def _matmul_nt(self, a, b, out=None, alpha=1.0, beta=0.0, row_scale=None):
        if self.gemm != "fp32":
            return matmul_nt(a, b, out=out, alpha=alpha, beta=beta, row_scale=row_scale,
                             two_planes=self.gemm == "split2")
        return gemm_nt(a, b, out=out, alpha=alpha, beta=beta, row_scale=row_scale)


_COPY_THREADS = 4
_pool = None


def _copy_pool():
    global _pool
    if _pool is None:
        from concurrent.futures import ThreadPoolExecutor

        _pool = ThreadPoolExecutor(_COPY_THREADS)
    return _pool


class ScoreAccumulator:
    """The checkpoint loop of TRAKer.finalize_scores (trak/traker.py:641-678) with the score sums
    kept on the GPU.

    The reference adds every checkpoint's [N, M] score matrix into a CPU tensor (one device-to-host
    copy of the whole matrix per checkpoint) and evaluates
    `(_scores / n) * (_avg_out_to_losses / n)` with numpy at the end.  Here `add` accumulates in the
    GEMM epilogue on the device, the out_to_loss sums stay a small host array exactly as in the
    reference, and `finalize` applies the same expression on the device while the matrix is
    written, chunk by chunk through page-locked memory, into the scores store: one crossing of
    PCIe in total.

    Args:
        score_computer: a BasicScoreComputer of this package.
        train_set_size, num_targets: N and M.
        dtype: torch.float16 or torch.float32, the saver's element type (trak/traker.py:127); it
            fixes the type the out_to_loss sums are kept in, as in the reference.
    """

    def __init__(self, score_computer, train_set_size, num_targets, dtype=ch.float32):
        import numpy as np

        self._np = np
        self.score_computer = score_computer
        self.shape = (int(train_set_size), int(num_targets))
        self.dtype = dtype
        self._acc = ch.zeros(self.shape, dtype=ch.float32, device=score_computer._dev)
        self._out_to_loss = np.zeros(
            (self.shape[0], 1), dtype=np.float16 if dtype == ch.float16 else np.float32
        )
        self.num_models = 0

    def add(self, features, target_grads, out_to_loss) -> None:
        """One checkpoint: sums += features @ target_grads^T (trak/traker.py:667) and
        out_to_loss sums += out_to_loss (trak/traker.py:670)."""
        self.score_computer.get_scores(features, target_grads, accumulator=self._acc)
        o = out_to_loss.detach().cpu().numpy() if isinstance(out_to_loss, Tensor) else self._np.asarray(out_to_loss)
        self._out_to_loss += o.reshape(self.shape[0], 1)
        self.num_models += 1

    def finalize(self, out, chunk_bytes: int = 256 << 20):
        """Writes `(sums / n) * (out_to_loss sums / n)` (trak/traker.py:674-676) into `out`, the
        [N, M] array behind the saver's `<exp>_scores` store (numpy array or memmap of float16 or
        float32) or a tensor (CUDA, or page-locked CPU).  Returns `out`."""
        np = self._np
        if self.num_models == 0:
            raise ValueError("no checkpoint was added")
        n = float(self.num_models)
        # the second factor exactly as numpy computes it in the reference, then widened (exact)
        row_factor = (self._out_to_loss / n).astype(np.float32).reshape(-1)
        row_factor = ch.from_numpy(row_factor).to(self._acc.device)
        N, M = self.shape
        if isinstance(out, Tensor):
            scores_finalize(self._acc, n, row_factor, out)
            if not out.is_cuda:
                ch.cuda.current_stream(self._acc.device).synchronize()
            return out
        if tuple(out.shape) != (N, M) or out.dtype not in (np.float16, np.float32):
            raise ValueError(f"out must be a [{N}, {M}] array of float16 or float32")
        tdtype = ch.float16 if out.dtype == np.float16 else ch.float32
        rows = max(1, min(N, int(chunk_bytes) // max(1, M * out.dtype.itemsize)))
        stage = [ch.empty((rows, M), dtype=tdtype).pin_memory() for _ in range(2 if rows < N else 1)]
        pending = [None] * len(stage)
        stream = ch.cuda.current_stream(self._acc.device)

        def retire(i):
            if pending[i] is None:
                return
            event, r0, r1 = pending[i]
            event.synchronize()
            # one thread copies about 30 GB/s, less than the 55 GB/s the kernel delivers over PCIe:
            # the copy into the store is spread over a few threads (numpy releases the GIL in it)
            src = stage[i][: r1 - r0].numpy()
            step = -(-(r1 - r0) // _COPY_THREADS)
            parts = [(a, min(r1 - r0, a + step)) for a in range(0, r1 - r0, step)]
            list(_copy_pool().map(lambda ab: out.__setitem__(slice(r0 + ab[0], r0 + ab[1]), src[ab[0] : ab[1]]), parts))
            pending[i] = None

        for index, r0 in enumerate(range(0, N, rows)):
            i = index % len(stage)
            retire(i)
            r1 = min(N, r0 + rows)
            scores_finalize(self._acc[r0:r1], n, row_factor[r0:r1], stage[i][: r1 - r0])
            event = ch.cuda.Event()
            event.record(stream)
            pending[i] = (event, r0, r1)
        for i in range(len(stage)):
            retire((index + 1 + i) % len(stage))
        return out
