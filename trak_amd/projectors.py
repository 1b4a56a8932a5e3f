"""Projector plug-ins with the interface of the reference's trak/projectors.py, computing on
an AMD GPU through libtrakhip.

`CudaProjector` and `ChunkedCudaProjector` keep the reference's names, constructor arguments
and `project` / `free_memory` methods (trak/projectors.py:317-516) so that
`TRAKer(projector=CudaProjector(...))` works unchanged ("cuda" is also how PyTorch-ROCm names
AMD devices).
"""
from abc import ABC, abstractmethod
from enum import Enum
from typing import Union

import torch
from torch import Tensor

from . import fast_jl
from .utils import vectorize

ch = torch


class ProjectionType(str, Enum):
    normal: str = "normal"
    rademacher: str = "rademacher"


class AbstractProjector(ABC):
    """Interface of trak/projectors.py:30-88."""

    @abstractmethod
    def __init__(
        self,
        grad_dim: int,
        proj_dim: int,
        seed: int,
        proj_type: Union[str, ProjectionType],
        device: Union[str, torch.device],
    ) -> None:
        self.grad_dim = grad_dim
        self.proj_dim = proj_dim
        self.seed = seed
        self.proj_type = proj_type
        self.device = device

    @abstractmethod
    def project(self, grads: Tensor, model_id: int) -> Tensor:
        """Projects a batch of gradients; model_id selects the projection matrix."""

    def free_memory(self):
        """Frees memory held by the projector."""


class NoOpProjector(AbstractProjector):
    """project(grads) = grads (trak/projectors.py:91-124)."""

    def __init__(self, grad_dim=0, proj_dim=0, seed=0, proj_type="na", device="cuda", *args, **kwargs):
        super().__init__(grad_dim, proj_dim, seed, proj_type, device)

    def project(self, grads, model_id):
        if isinstance(grads, dict):
            grads = vectorize(grads, device=self.device)
        return grads

    def free_memory(self):
        pass


def _type_name(proj_type):
    name = proj_type.value if isinstance(proj_type, ProjectionType) else str(proj_type)
    if name not in ("normal", "rademacher"):
        raise KeyError(f"Projection type {proj_type} not recognized.")
    return name


class CudaProjector(AbstractProjector):
    """On-the-fly JL projection on the GPU (trak/projectors.py:317-427)."""

    def __init__(
        self,
        grad_dim: int,
        proj_dim: int,
        seed: int,
        proj_type: ProjectionType,
        device,
        max_batch_size: int,
        *args,
        **kwargs,
    ) -> None:
        """
        Args match the reference.  max_batch_size (8, 16 or 32) only selects which of the
        `project_<type>_<n>` entry points is called; all of them give the same result here.
        kwargs may carry num_sms to pin the number of feature tiles (the projection matrix
        depends on it, as in the reference; default = the device's compute-unit count).

        Raises:
            ValueError: on a non-CUDA device.
            ModuleNotFoundError: when libtrakhip is not built.
        """
        super().__init__(grad_dim, proj_dim, seed, proj_type, device)
        self.max_batch_size = max_batch_size

        if isinstance(device, str):
            device = ch.device(device)
        if device.type != "cuda":
            raise ValueError(
                "CudaProjector only works on a CUDA device; Either switch to a CUDA device, or use the BasicProjector"
            )
        index = device.index if device.index is not None else ch.cuda.current_device()
        self._device = ch.device("cuda", index)
        num_sms = kwargs.get("num_sms")
        if num_sms is None:
            num_sms = ch.cuda.get_device_properties(index).multi_processor_count
        self.num_sms = int(num_sms)

        try:
            # test run to catch at init time if projection goes through (trak/projectors.py:372-378)
            fast_jl.project_rademacher_8(ch.zeros(8, 1_000, device=self._device), 512, 0, self.num_sms)
        except ImportError:
            raise ModuleNotFoundError(
                "libtrakhip.so is not built; run `python -m trak_amd.build` (see the installation notes)."
            )

    def project(self, grads: Union[dict, Tensor], model_id: int) -> Tensor:
        if isinstance(grads, dict):
            tensors = list(grads.values())
            if fast_jl.gather_supported(tensors) and tensors[0].device == self._device:
                # the kernel reads the per-parameter tensors in place: same result as projecting
                # vectorize(grads) (trak/projectors.py:389-390) without building the [B, P] copy
                return fast_jl.project_gather(
                    tensors, self.proj_dim, self.seed + int(1e4) * model_id, self.num_sms, _type_name(self.proj_type)
                )
            grads = vectorize(grads, device=self.device)

        batch_size = grads.shape[0]
        effective_batch_size = 32
        if batch_size <= 8:
            effective_batch_size = 8
        elif batch_size <= 16:
            effective_batch_size = 16
        effective_batch_size = min(self.max_batch_size, effective_batch_size)

        fn = getattr(fast_jl, f"project_{_type_name(self.proj_type)}_{effective_batch_size}")
        return fn(grads, self.proj_dim, self.seed + int(1e4) * model_id, self.num_sms)

    def project_into(self, grads: Union[dict, Tensor], model_id: int, out: Tensor, scale: float = 1.0) -> Tensor:
        """out[B, proj_dim] = cast(project(grads, model_id) * scale), written by the kernel that sums
        the feature tiles: `out` is a CUDA tensor or a page-locked CPU tensor of fp16 / bf16 / fp32.
        Covers `project` plus `grads /= normalize_factor; grads.to(dtype).cpu()` of
        trak/traker.py:425-428 (scale = 1 / normalize_factor).  Work is only enqueued: synchronize
        before reading a CPU destination."""
        if isinstance(grads, dict):
            tensors = list(grads.values())
            if fast_jl.gather_supported(tensors) and tensors[0].device == self._device:
                source = tensors
            else:
                source = vectorize(grads, device=self.device)
        else:
            source = grads
        return fast_jl.project_into(
            source, self.proj_dim, self.seed + int(1e4) * model_id, self.num_sms, _type_name(self.proj_type), out, scale
        )

    def free_memory(self):
        """A no-op method."""


class ChunkedCudaProjector:
    """Projects a gradient dict whose parameters were grouped into chunks, one CudaProjector per
    chunk, and sums the chunk projections (trak/projectors.py:430-516)."""

    def __init__(
        self,
        projector_per_chunk: list,
        max_chunk_size: int,
        params_per_chunk: list,
        feat_bs: int,
        device: torch.device,
        dtype: torch.dtype,
        accumulate_in_dtype: bool = False,
    ):
        # accumulate_in_dtype=True reproduces the reference's arithmetic to the bit: the running sum of
        # the chunk projections is kept in `dtype` and rounded after every addition
        # (trak/projectors.py:472-474, :490-495, :509-514).  The default keeps the sum in fp32 and rounds
        # once at the end, which is at least as accurate and what the kernels produce anyway.
        self.accumulate_in_dtype = accumulate_in_dtype
        self.projector_per_chunk = projector_per_chunk
        self.proj_dim = self.projector_per_chunk[0].proj_dim
        self.proj_type = self.projector_per_chunk[0].proj_type
        self.params_per_chunk = params_per_chunk

        self.max_chunk_size = max_chunk_size
        self.feat_bs = feat_bs
        self.device = device
        self.dtype = dtype
        self.input_allocated = False

    def allocate_input(self):
        """Kept for interface compatibility (trak/projectors.py:452-462 allocates a
        [feat_bs, max_chunk_size] packing buffer here): nothing is packed in this implementation, the
        chunks are projected where the gradients are."""
        self.input_allocated = True

    def free_memory(self):
        self.input_allocated = False

    def _chunk_sizes(self, grads):
        """Greedy grouping of the dict's parameters into chunks of at most max_chunk_size features,
        in dict order - the rule of trak/projectors.py:479-503 and of get_parameter_chunk_sizes
        (trak/utils.py:297-331).  Returns [(first parameter index, end index, features)]."""
        groups, begin, width = [], 0, 0
        for i, p in enumerate(grads.values()):
            param_size = 1 if len(p.shape) < 2 else p[0].numel()
            if width + param_size > self.max_chunk_size:
                groups.append((begin, i, width))
                begin, width = i, 0
            width += param_size
        groups.append((begin, len(grads), width))
        got = [g[2] for g in groups]
        assert got == [int(x) for x in self.params_per_chunk], (got, list(self.params_per_chunk))
        return groups

    def _accumulate(self, parts, rows):
        """Sum of the chunk projections (fp32 each, as fast_jl returns them), returned in `dtype`."""
        if self.accumulate_in_dtype:
            acc = ch.zeros(size=(rows, self.proj_dim), device=self.device, dtype=self.dtype)
            for part in parts:
                acc.add_(part)  # fp32 + dtype -> rounded to dtype after every chunk, as the reference does
            return acc
        acc = None
        for part in parts:
            acc = part.to(ch.float32) if acc is None else acc.add_(part)
        return acc.to(self.dtype)

    def project(self, grads, model_id):
        names = list(grads.keys())
        tensors = list(grads.values())
        rows = tensors[0].shape[0]
        if rows > self.feat_bs:
            # the reference's packing buffer has feat_bs rows: a larger batch fails on its copy_
            # (trak/projectors.py:500-502)
            raise RuntimeError(f"batch of {rows} rows exceeds feat_bs = {self.feat_bs}")
        groups = self._chunk_sizes(grads)
        if fast_jl.gather_supported(tensors) and tensors[0].dtype == self.dtype:
            # every chunk goes to its projector as a dict, which projects the tensors where they are
            parts = (
                self.projector_per_chunk[i].project({n: grads[n] for n in names[b:e]}, model_id=model_id)
                for i, (b, e, _) in enumerate(groups)
            )
            return self._accumulate(parts, rows)
        # mixed dtypes or host tensors: one flat [rows, P] copy in `dtype` (what the reference's packing
        # buffer holds after its copy_), projected chunk by chunk through column slices
        flat = vectorize({n: t.to(self.dtype) for n, t in grads.items()}, device=self.device)
        edges = [0]
        for _, _, width in groups:
            edges.append(edges[-1] + width)
        parts = (
            self.projector_per_chunk[i].project(flat[:, edges[i]:edges[i + 1]], model_id=model_id)
            for i in range(len(groups))
        )
        return self._accumulate(parts, rows)
