"""The store side of TRAKer.featurize: projected gradients go from the projection kernel into a
page-locked staging buffer and from there into the `grads` rows of the saver's store.

In the reference this is (trak/traker.py:425-429)

    grads = self.projector.project(grads, model_id=...)
    grads /= self.normalize_factor
    self.saver.current_store["grads"][inds] = grads.to(self.dtype).cpu().clone().detach()

i.e. a scaling pass, a cast pass, a blocking device-to-host copy and a host copy per batch.
`FeatureWriter.write` does the same with one kernel (scale and cast happen where the feature
tiles are summed, the result is written over PCIe into pinned memory) and without stalling the
GPU: a batch is copied into the store when its slot of the staging ring is needed again, or at
`flush`.  Stored values are identical, bit for bit, to the reference sequence.
"""
import numpy as np
import torch

_NP_DTYPES = {torch.float16: np.float16, torch.float32: np.float32}


class FeatureWriter:
    """Ring of page-locked [max_batch_size, proj_dim] buffers between a projector and a store.

    Args:
        projector: a projector of this package (or anything with `project(grads, model_id)`).
        proj_dim: number of JL dimensions (columns of the store).
        normalize_factor: the divisor of trak/traker.py:426 (sqrt of the parameter count).
        dtype: torch.float16 or torch.float32, the store's element type (trak/traker.py:127).
        max_batch_size: most rows one `write` may carry.
        depth: number of staging buffers = batches that may be in flight.
    """

    def __init__(self, projector, proj_dim, normalize_factor, dtype=torch.float32, max_batch_size=32, depth=2):
        if dtype not in _NP_DTYPES:
            raise ValueError("the store's dtype must be torch.float16 or torch.float32")
        if depth < 1:
            raise ValueError("depth must be at least 1")
        self.projector = projector
        self.proj_dim = int(proj_dim)
        self.dtype = dtype
        # torch divides a CUDA tensor by a CPU scalar as a multiplication by the fp32 reciprocal
        self.normalize_factor = torch.as_tensor(normalize_factor, dtype=torch.float32).reshape(()).cpu()
        self.scale = float(torch.ones((), dtype=torch.float32) / self.normalize_factor)
        self.max_batch_size = int(max_batch_size)
        self._slots = [
            torch.empty((self.max_batch_size, self.proj_dim), dtype=dtype).pin_memory() for _ in range(depth)
        ]
        self._pending = [None] * depth  # (event, store, inds, rows)
        self._next = 0

    def _retire(self, i):
        item = self._pending[i]
        if item is None:
            return
        event, store, inds, rows = item
        event.synchronize()
        store[inds] = self._slots[i][:rows].numpy()
        self._pending[i] = None

    def write(self, grads, model_id, store, inds):
        """Projects `grads` (tensor [B, P] or per-parameter dict) and schedules
        `store[inds] = projection / normalize_factor` in the store's dtype.  `store` is the array
        behind `saver.current_store["grads"]` (any object with numpy item assignment); `inds` as in
        the reference (index array of B rows).  The rows are in the store after `flush()`."""
        i = self._next
        self._next = (i + 1) % len(self._slots)
        self._retire(i)
        first = next(iter(grads.values())) if isinstance(grads, dict) else grads
        rows = int(first.shape[0])
        if rows > self.max_batch_size:
            raise ValueError(f"batch of {rows} rows exceeds max_batch_size={self.max_batch_size}")
        slot = self._slots[i][:rows]
        device = first.device
        if hasattr(self.projector, "project_into"):
            self.projector.project_into(grads, model_id, slot, self.scale)
        else:
            # any other projector: the reference's sequence of passes, with an asynchronous copy
            projected = self.projector.project(grads, model_id=model_id)
            projected = projected / self.normalize_factor
            slot.copy_(projected.to(self.dtype), non_blocking=True)
            device = projected.device
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream(device))
        self._pending[i] = (event, store, inds, rows)

    def flush(self):
        """Waits for every batch in flight and copies it into its store."""
        n = len(self._slots)
        for step in range(n):
            self._retire((self._next + step) % n)
