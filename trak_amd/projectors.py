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
    ):
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
        if self.input_allocated:
            return
        # the widest chunk that will actually be packed (the reference allocates max_chunk_size
        # columns, i.e. always close to 2^32 / feat_bs elements per row)
        width = int(max(self.params_per_chunk))
        self.ch_input = ch.zeros(size=(self.feat_bs, width), device=self.device, dtype=self.dtype)
        self.input_allocated = True

    def free_memory(self):
        if not self.input_allocated:
            return
        del self.ch_input
        self.input_allocated = False

    def _project_in_place(self, grads, model_id):
        """Same grouping rule as the packing path below, but every chunk is handed to its projector
        as a dict, which projects the parameter tensors where they are."""
        groups, current, pointer = [], {}, 0
        for name, p in grads.items():
            param_size = 1 if len(p.shape) < 2 else p[0].numel()
            if pointer + param_size > self.max_chunk_size:
                groups.append((current, pointer))
                current, pointer = {}, 0
            current[name] = p
            pointer += param_size
        groups.append((current, pointer))
        actual_bs = min(self.feat_bs, next(iter(grads.values())).shape[0])
        acc = None
        for index, (group, size) in enumerate(groups):
            assert size == self.params_per_chunk[index]
            if actual_bs != next(iter(group.values())).shape[0]:
                group = {k: v[:actual_bs] for k, v in group.items()}
            part = self.projector_per_chunk[index].project(group, model_id=model_id)
            acc = part if acc is None else acc.add_(part)
        return acc.to(self.dtype)

    def project(self, grads, model_id):
        tensors = list(grads.values())
        if fast_jl.gather_supported(tensors) and tensors[0].dtype == self.dtype:
            return self._project_in_place(grads, model_id)
        self.allocate_input()
        acc = ch.zeros(size=(self.feat_bs, self.proj_dim), device=self.device, dtype=ch.float32)
        pointer = 0
        projector_index = 0
        actual_bs = 0
        for p in grads.values():
            if len(p.shape) < 2:
                p_flat = p.data.unsqueeze(-1)
            else:
                p_flat = p.data.flatten(start_dim=1)

            param_size = p_flat.size(1)
            if pointer + param_size > self.max_chunk_size:
                assert pointer == self.params_per_chunk[projector_index]
                # the kernel takes the row pitch, so the packed prefix is projected in place
                acc[:actual_bs].add_(
                    self.projector_per_chunk[projector_index].project(
                        self.ch_input[:actual_bs, :pointer], model_id=model_id
                    )
                )
                pointer = 0
                projector_index += 1

            actual_bs = min(self.ch_input.size(0), p_flat.size(0))
            self.ch_input[:actual_bs, pointer : pointer + param_size].copy_(p_flat)
            pointer += param_size

        assert pointer == self.params_per_chunk[projector_index]
        acc[:actual_bs].add_(
            self.projector_per_chunk[projector_index].project(
                self.ch_input[:actual_bs, :pointer], model_id=model_id
            )
        )
        return acc[:actual_bs].to(self.dtype)
