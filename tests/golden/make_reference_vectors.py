#!/usr/bin/env python3
"""Writes tests/golden/reference_vectors.npz: small input/output vectors of the reference's own
CPU-runnable code for the functions of the hot path that no closed form pins by value:
BasicProjector (its matrix comes from torch's CPU generator), vectorize,
get_parameter_chunk_sizes and BasicScoreComputer.

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
out["torch_version"] = np.array(torch.__version__)

path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "reference_vectors.npz")
np.savez_compressed(path, **out)
print("wrote", path, {k: getattr(v, "shape", None) for k, v in out.items()})
