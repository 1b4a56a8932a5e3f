"""Host-side mirror of the reference's projector helpers (no GPU needed)."""
import pytest
import torch

from trak_amd import ChunkedCudaProjector, CudaProjector, NoOpProjector, ProjectionType, fast_jl, vectorize
from trak_amd.utils import chunk_sizes_from_numels, get_matrix_mult, get_parameter_chunk_sizes


def test_projection_type_enum():
    # trak/projectors.py:25-27
    assert ProjectionType.normal.value == "normal" and ProjectionType.rademacher.value == "rademacher"
    assert ProjectionType("normal") is ProjectionType.normal and isinstance(ProjectionType.normal, str)


def test_vectorize_dict_order_and_low_rank_params():
    # trak/utils.py:80-110: dict order, params with < 2 dims become one column
    g = {
        "w": torch.arange(2 * 3 * 4, dtype=torch.float32).reshape(2, 3, 4),
        "s": torch.tensor([100.0, 200.0]),
        "b": torch.arange(2 * 5, dtype=torch.float32).reshape(2, 5) + 1000,
    }
    out = vectorize(g, device="cpu")
    assert out.shape == (2, 12 + 1 + 5)
    assert torch.equal(out[:, :12], g["w"].reshape(2, 12))
    assert torch.equal(out[:, 12], g["s"])
    assert torch.equal(out[:, 13:], g["b"])
    arr = torch.zeros(2, 18)
    assert vectorize(g, arr=arr, device="cpu") is arr and torch.equal(arr, out)


def test_chunk_sizes_follow_the_uint32_rule():
    # trak/utils.py:297-331: max_chunk_size = uint32.max // batch_size, greedy grouping
    mx, per = chunk_sizes_from_numels([10, 20, 30], 32)
    assert mx == 4294967295 // 32 == 134217727 and per == [60]
    sizes = [60_000_000, 60_000_000, 60_000_000, 5]
    mx, per = chunk_sizes_from_numels(sizes, 32)
    assert per == [120_000_000, 60_000_005] and sum(per) == sum(sizes)
    mx, per = chunk_sizes_from_numels([100, 100], 4294967295 // 150)
    assert mx == 150 and per == [100, 100]
    model = torch.nn.Sequential(torch.nn.Linear(10, 7), torch.nn.Linear(7, 3))
    mx, per = get_parameter_chunk_sizes(model, 8)
    assert mx == 4294967295 // 8 and per == [10 * 7 + 7 + 7 * 3 + 3]


def test_cuda_projector_rejects_cpu_device():
    # trak/projectors.py:363-365
    with pytest.raises(ValueError, match="only works on a CUDA device"):
        CudaProjector(grad_dim=10, proj_dim=512, seed=0, proj_type=ProjectionType.rademacher, device="cpu", max_batch_size=8)


def test_noop_projector():
    p = NoOpProjector()
    g = torch.randn(3, 7)
    assert p.project(g, model_id=0) is g
    p.free_memory()


def test_fast_jl_namespace_and_input_checks():
    # the six entry points of fast_jl/fast_jl.cu:102-110
    for t in ("rademacher", "normal"):
        for n in (8, 16, 32):
            assert callable(getattr(fast_jl, f"project_{t}_{n}"))
    x = torch.zeros(8, 1000)
    with pytest.raises(RuntimeError, match="CUDA tensor"):   # fast_jl/fast_jl.cu:21
        fast_jl.project_rademacher_8(x, 512, 0, 256)


def test_get_matrix_mult_cpu_path_is_plain_matmul():
    a, b = torch.randn(5, 8), torch.randn(3, 8)
    out = get_matrix_mult(a, b)
    assert out.shape == (5, 3) and torch.allclose(out, a @ b.t())


def test_chunked_projector_bookkeeping_with_a_fake_chunk_projector():
    # packing order, flush rule and summation of trak/projectors.py:470-516, checked on the CPU
    # with a stand-in for the per-chunk projector
    class Fake:
        proj_dim, proj_type = 4, ProjectionType.rademacher

        def __init__(self, scale):
            self.scale, self.seen = scale, []

        def project(self, grads, model_id):
            self.seen.append(grads.clone())
            return torch.full((grads.shape[0], 4), float(grads.sum()) * self.scale)

    fakes = [Fake(1.0), Fake(10.0)]
    proj = ChunkedCudaProjector(fakes, max_chunk_size=7, params_per_chunk=[7, 4], feat_bs=3, device="cpu", dtype=torch.float32)
    g = {"a": torch.ones(2, 2, 2), "b": torch.ones(2, 2) * 2, "c": torch.ones(2) * 3, "d": torch.ones(2, 4) * 5}
    out = proj.project(g, model_id=0)
    assert out.shape == (2, 4)
    assert fakes[0].seen[0].shape == (2, 7) and fakes[1].seen[0].shape == (2, 4)
    assert torch.equal(fakes[0].seen[0][0], torch.tensor([1.0, 1, 1, 1, 2, 2, 3]))
    assert torch.equal(fakes[1].seen[0][0], torch.tensor([5.0, 5, 5, 5]))
    assert torch.allclose(out, torch.full((2, 4), 2 * 11.0 + 10 * 2 * 20.0))
    proj.free_memory()
    assert not proj.input_allocated
