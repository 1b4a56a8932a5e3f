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


@pytest.mark.parametrize("tag,dt", [("fp16", torch.float16), ("bf16", torch.bfloat16)])
def test_chunked_accumulation_in_dtype_matches_reference_vectors(tag, dt):
    # The reference's ChunkedCudaProjector adds the fp32 chunk projections into an accumulator of its
    # `dtype`, rounding after every chunk (trak/projectors.py:472-495).  accumulate_in_dtype=True must
    # give its bits; the default (fp32 sum, one rounding) must be the correctly rounded sum instead.
    from trak_amd import ChunkedCudaProjector

    grads = {k: torch.from_numpy(GOLD[f"chunk_in_{k}"]).to(dt) for k in ("a", "b", "c", "d")}
    sizes = [701, 300]
    per = [BasicProjectorCPU(grad_dim=sz, proj_dim=128, seed=3 + i, proj_type="rademacher") for i, sz in enumerate(sizes)]
    exact = ChunkedCudaProjector(per, 750, sizes, 4, "cpu", dt, accumulate_in_dtype=True).project(grads, model_id=0)
    assert exact.dtype == dt and exact.shape == (3, 128)
    assert np.array_equal(exact.float().numpy(), GOLD[f"chunk_out_{tag}"])
    default = ChunkedCudaProjector(per, 750, sizes, 4, "cpu", dt).project(grads, model_id=0)
    flat = vectorize(grads, device="cpu")
    parts = [per[0].project(flat[:, :701], model_id=0), per[1].project(flat[:, 701:], model_id=0)]
    assert torch.equal(default, (parts[0] + parts[1]).to(dt))
    # the two differ by the extra rounding of the first chunk's part: at most one step of dt at its size
    step = torch.finfo(dt).eps * torch.maximum(parts[0].abs(), default.float().abs())
    assert ((exact.float() - default.float()).abs() <= step).all()
    assert not torch.equal(exact, default)
    # a batch larger than feat_bs is refused (the reference fails on its packing copy)
    big = {k: torch.cat([v, v]) for k, v in grads.items()}
    with pytest.raises(RuntimeError, match="feat_bs"):
        ChunkedCudaProjector(per, 750, sizes, 4, "cpu", dt).project(big, model_id=0)


@pytest.mark.gpu
def test_gpu_score_computer_fp16_in_dtype_matches_reference_vectors(gpu):
    # fp16 `dtype`, three row blocks: the reference rounds every block product and the running sum to
    # fp16 and adds lambda in fp16 (trak/score_computers.py:147-162).  Its CPU matmul and this GPU one
    # add the 50 products of a block in different orders, so single entries may land on the other side
    # of an fp16 rounding boundary: at most one fp16 step apart, and nearly all identical.
    from trak_amd import BasicScoreComputer

    X = torch.from_numpy(GOLD["sch_X"]).half()
    want_xtx, want_f = GOLD["sch_xtx"], GOLD["sch_features"]
    sc = BasicScoreComputer(dtype=torch.float16, device="cuda:0", CUDA_MAX_DIM_SIZE=50, lambda_reg=1e-2,
                            accumulate_in_dtype=True)
    xtx = sc.get_xtx(X)
    assert xtx.dtype == torch.float16
    got = xtx.float().cpu().numpy()
    step = np.maximum(np.abs(want_xtx), 2.0**-14) * 2.0**-10
    assert np.all(np.abs(got - want_xtx) <= step)
    assert np.mean(got == want_xtx) > 0.9
    feats = sc.get_x_xtx_inv(X, xtx)
    assert feats.dtype == torch.float16
    rel = np.abs(feats.float().cpu().numpy() - want_f).max() / np.abs(want_f).max()
    assert rel < 5e-3
    # the default (fp32 sums, one rounding) is the more accurate of the two against float64
    sc32 = BasicScoreComputer(dtype=torch.float16, device="cuda:0", CUDA_MAX_DIM_SIZE=50, lambda_reg=1e-2)
    x64 = GOLD["sch_X"].astype(np.float64)
    truth = x64.T @ x64
    err_default = np.abs(sc32.get_xtx(X).float().cpu().numpy() - truth).max()
    err_exact = np.abs(got - truth).max()
    assert err_default <= err_exact + 1e-12
