#!/usr/bin/env python3
"""Writes tests/golden/reference_vectors.npz: small input/output vectors of the reference's own
CPU-runnable code for the functions of the hot path that no closed form pins by value:
BasicProjector (its matrix comes from torch's CPU generator), vectorize,
get_parameter_chunk_sizes, BasicScoreComputer (fp32 and fp16) and ChunkedCudaProjector's accumulation.

Run once, in the container that has the reference checked out at /root/reference:
    python tests/golden/make_reference_vectors.py
Only the vectors are committed; the reference itself never travels.
"""
import os
import sys

import numpy as np
import torch

REFERENCE = os.environ.get("TRAK_REFERENCE", "/root/reference")
sys.path.insert(0, REFERENCE)

from trak.projectors import BasicProjector, ProjectionType  # noqa: E402
from trak.score_computers import BasicScoreComputer  # noqa: E402
from trak.utils import get_parameter_chunk_sizes, vectorize  # noqa: E402

out = {}
gen = torch.Generator().manual_seed(1234)

# BasicProjector: rademacher and normal, several blocks (proj_dim 250 -> blocks of 100, 100, 50)
g = torch.randn(3, 700, generator=gen)
out["bp_grads"] = g.numpy()
for name, pt in (("rademacher", ProjectionType.rademacher), ("normal", ProjectionType.normal)):
    p = BasicProjector(grad_dim=700, proj_dim=250, seed=5, proj_type=pt, device="cpu")
    out[f"bp_{name}_model0"] = p.project(g, model_id=0).numpy()
    out[f"bp_{name}_model2"] = p.project(g, model_id=2).numpy()
p1 = BasicProjector(grad_dim=700, proj_dim=64, seed=9, proj_type=ProjectionType.rademacher, device="cpu")
out["bp_single_block"] = p1.project(g, model_id=0).numpy()

# vectorize
grads = {
    "w": torch.randn(2, 3, 4, generator=gen),
    "s": torch.randn(2, generator=gen),
    "b": torch.randn(2, 5, generator=gen),
}
for k, v in grads.items():
    out[f"vec_in_{k}"] = v.numpy()
out["vec_out"] = vectorize(grads, device="cpu").numpy()

# get_parameter_chunk_sizes on a small model with an artificially small limit
model = torch.nn.Sequential(torch.nn.Linear(40, 30), torch.nn.Linear(30, 20), torch.nn.Linear(20, 5))
bs = int(np.iinfo(np.uint32).max // 1500)
mx, per = get_parameter_chunk_sizes(model, bs)
out["chunks_numels"] = np.array([p.numel() for p in model.parameters()])
out["chunks_batch_size"] = np.array(bs)
out["chunks_max"] = np.array(mx)
out["chunks_per"] = np.array(per)

# BasicScoreComputer on the CPU
X = torch.randn(130, 16, generator=gen) / 4
Xt = torch.randn(11, 16, generator=gen) / 4
sc = BasicScoreComputer(dtype=torch.float32, device="cpu", CUDA_MAX_DIM_SIZE=50, lambda_reg=1e-2)
xtx = sc.get_xtx(X)
feats = sc.get_x_xtx_inv(X, xtx)
acc = torch.zeros(130, 11)
sc.get_scores(feats, Xt, acc)
out["sc_X"], out["sc_Xt"] = X.numpy(), Xt.numpy()
out["sc_xtx"], out["sc_features"], out["sc_scores"] = xtx.numpy(), feats.numpy(), acc.numpy()
# ChunkedCudaProjector: the reference's class, driven with CPU BasicProjectors in place of
# CudaProjectors (both return fp32 parts for the packed chunk), with a 16-bit `dtype`: pins how the
# chunk projections are accumulated (in `dtype`, rounded after every chunk: trak/projectors.py:472-495)
from trak.projectors import ChunkedCudaProjector  # noqa: E402

cg = {
    "a": torch.randn(3, 40, 10, generator=gen) * 0.7,
    "b": torch.randn(3, 300, generator=gen) * 0.7,
    "c": torch.randn(3, generator=gen),
    "d": torch.randn(3, 25, 12, generator=gen) * 0.7,
}
sizes = [400 + 300 + 1, 300]          # "d" does not fit next to the first three under a limit of 750
for k_, v in cg.items():
    out[f"chunk_in_{k_}"] = v.numpy()
for tag, dt in (("fp16", torch.float16), ("bf16", torch.bfloat16)):
    per = [BasicProjector(grad_dim=sz, proj_dim=128, seed=3 + i, proj_type=ProjectionType.rademacher,
                          device="cpu", dtype=torch.float32) for i, sz in enumerate(sizes)]
    cp = ChunkedCudaProjector(per, 750, sizes, 4, "cpu", dt)
    res = cp.project({k_: v.to(dt) for k_, v in cg.items()}, model_id=0)
    assert res.dtype == dt and res.shape == (3, 128)
    out[f"chunk_out_{tag}"] = res.float().numpy()

# BasicScoreComputer with a 16-bit dtype and three row blocks: pins the per-block rounding of X^T X,
# lambda added in the 16-bit type and the type of the returned features (trak/score_computers.py:145-177)
Xh = (torch.randn(130, 16, generator=gen) / 2).half()
sch = BasicScoreComputer(dtype=torch.float16, device="cpu", CUDA_MAX_DIM_SIZE=50, lambda_reg=1e-2)
xtx_h = sch.get_xtx(Xh)
feats_h = sch.get_x_xtx_inv(Xh, xtx_h)
assert xtx_h.dtype == torch.float16 and feats_h.dtype == torch.float16
out["sch_X"], out["sch_xtx"], out["sch_features"] = Xh.float().numpy(), xtx_h.float().numpy(), feats_h.float().numpy()
out["torch_version"] = np.array(torch.__version__)

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
np.savez_compressed(path, **out)
print("wrote", path, {k: getattr(v, "shape", None) for k, v in out.items()})
