"""TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's BasicProjector
(trak/projectors.py:209-314), the projector TRAK itself falls back to on a CPU
(trak/traker.py:244-251).  It is the `cpu_baseline` that bench.py times next to the GPU
kernel, and a statistical cross-check in the tests.  Its random matrix comes from torch's
CPU generator, so its values differ from the GPU path's Philox stream by construction; the
two are compared through JL properties only.

Pinned by: the block-seed closed form seed + 1000*i + 100000*model_id
(trak/projectors.py:262-267), determinism under re-seeding, entries in {-1,+1} /
unit-variance normals, and norm preservation (tests/test_oracle_baselines.py).
"""
import math

import torch


class BasicProjectorCPU:
    def __init__(self, grad_dim, proj_dim, seed, proj_type, block_size=100, dtype=torch.float32, model_id=0):
        self.grad_dim = grad_dim
        self.proj_dim = proj_dim
        self.seed = seed
        self.proj_type = getattr(proj_type, "value", proj_type)
        self.block_size = min(proj_dim, block_size)           # trak/projectors.py:240
        self.num_blocks = math.ceil(proj_dim / self.block_size)  # :241
        self.dtype = dtype
        self.model_id = model_id
        self.proj_matrix = torch.empty(grad_dim, self.block_size, dtype=dtype)
        self.generator = torch.Generator(device="cpu")

    def block_seeds(self, model_id=None):
        mid = self.model_id if model_id is None else model_id
        return [self.seed + 1000 * i + 100000 * mid for i in range(self.num_blocks)]  # :262-264

    def generate_block(self, block_seed):
        self.generator.manual_seed(block_seed)
        if self.proj_type == "normal":
            self.proj_matrix.normal_(generator=self.generator)       # :279
        elif self.proj_type == "rademacher":
            self.proj_matrix.bernoulli_(p=0.5, generator=self.generator)  # :284
            self.proj_matrix *= 2.0
            self.proj_matrix -= 1.0
        else:
            raise KeyError(f"Projection type {self.proj_type} not recognized.")
        return self.proj_matrix

    def project(self, grads, model_id=0, max_blocks=None):
        """grads [B, P] -> sketch [B, proj_dim] (trak/projectors.py:290-314).  max_blocks limits
        the number of 100-column blocks computed (for timing a sample); the rest stay zero."""
        grads = grads.to(self.dtype)
        sketch = torch.zeros(grads.size(0), self.proj_dim, dtype=self.dtype)
        seeds = self.block_seeds(model_id)
        nblocks = self.num_blocks if max_blocks is None else min(max_blocks, self.num_blocks)
        for ind in range(nblocks):
            m = self.generate_block(seeds[ind])
            st = ind * self.block_size
            ed = min((ind + 1) * self.block_size, self.proj_dim)
            sketch[:, st:ed] = grads @ m[:, : ed - st]
        return sketch
