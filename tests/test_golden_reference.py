"""Checks against tests/golden/reference_vectors.npz: outputs of the reference's own CPU code
(written by tests/golden/make_reference_vectors.py) for BasicProjector, vectorize,
get_parameter_chunk_sizes and BasicScoreComputer."""
import os

import numpy as np
import pytest
import torch

from oracle import score_oracle as so
from oracle.basic_projector import BasicProjectorCPU
from trak_amd import vectorize
from trak_amd.utils import chunk_sizes_from_numels

GOLD = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "reference_vectors.npz"))


@pytest.mark.parametrize("name", ["rademacher", "normal"])
def test_basic_projector_restatement_matches_reference_vectors(name):
    g = torch.from_numpy(GOLD["bp_grads"])
    p = BasicProjectorCPU(grad_dim=700, proj_dim=250, seed=5, proj_type=name)
    for mid in (0, 2):
        got = p.project(g, model_id=mid).numpy()
        np.testing.assert_allclose(got, GOLD[f"bp_{name}_model{mid}"], rtol=1e-5, atol=1e-4)


def test_basic_projector_single_block_matches_reference_vectors():
    g = torch.from_numpy(GOLD["bp_grads"])
    p = BasicProjectorCPU(grad_dim=700, proj_dim=64, seed=9, proj_type="rademacher")
    np.testing.assert_allclose(p.project(g, model_id=0).numpy(), GOLD["bp_single_block"], rtol=1e-5, atol=1e-4)


def test_vectorize_matches_reference_vectors():
    grads = {k: torch.from_numpy(GOLD[f"vec_in_{k}"]) for k in ("w", "s", "b")}
    assert np.array_equal(vectorize(grads, device="cpu").numpy(), GOLD["vec_out"])


def test_chunk_sizes_match_reference_vectors():
    mx, per = chunk_sizes_from_numels(GOLD["chunks_numels"].tolist(), int(GOLD["chunks_batch_size"]))
    assert mx == int(GOLD["chunks_max"]) and per == GOLD["chunks_per"].tolist()
    assert len(per) == 2   # the vector exercises a real split


def test_score_oracles_match_reference_vectors():
    X, Xt = GOLD["sc_X"], GOLD["sc_Xt"]
    cpu = so.BasicScoreComputerCPU(lambda_reg=1e-2, max_dim=50)
    xtx = cpu.get_xtx(torch.from_numpy(X))
    np.testing.assert_allclose(xtx.numpy(), GOLD["sc_xtx"], rtol=1e-5, atol=1e-6)
    feats = cpu.get_x_xtx_inv(torch.from_numpy(X), xtx)
    np.testing.assert_allclose(feats.numpy(), GOLD["sc_features"], rtol=1e-4, atol=1e-5)
    acc = torch.zeros(130, 11)
    cpu.get_scores(feats, torch.from_numpy(Xt), acc)
    np.testing.assert_allclose(acc.numpy(), GOLD["sc_scores"], rtol=1e-4, atol=1e-5)
    # the float64 oracle agrees with the reference's float32 result to float32 accuracy
    f64, _, _ = so.x_xtx_inv_f64(X, so.xtx_f64(X), 1e-2)
    s64 = so.scores_f64(f64, Xt)
    assert np.abs(s64 - GOLD["sc_scores"]).max() / np.abs(s64).max() < 1e-4


@pytest.mark.gpu
def test_gpu_score_computer_matches_reference_vectors(gpu):
    from trak_amd import BasicScoreComputer

    X, Xt = torch.from_numpy(GOLD["sc_X"]), torch.from_numpy(GOLD["sc_Xt"])
    sc = BasicScoreComputer(dtype=torch.float32, device="cuda:0", CUDA_MAX_DIM_SIZE=50, lambda_reg=1e-2)
    xtx = sc.get_xtx(X)
    feats = sc.get_x_xtx_inv(X, xtx)
    acc = torch.zeros(130, 11)
    sc.get_scores(feats, Xt.to(gpu), acc)
    rel = lambda a, b: np.abs(a - b).max() / np.abs(b).max()
    assert rel(xtx.cpu().numpy(), GOLD["sc_xtx"]) < 1e-5
    assert rel(feats.cpu().numpy(), GOLD["sc_features"]) < 1e-4
    assert rel(acc.numpy(), GOLD["sc_scores"]) < 1e-4
