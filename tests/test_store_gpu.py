"""GPU tests of the store-side epilogues: the projection's scale + cast + write into page-locked
memory (TRAKer.featurize, trak/traker.py:425-429), the score finalization
(trak/traker.py:670-678) and the two host classes that drive them.  The bar is bit equality with
the reference's own sequence of torch / numpy operations on the same projected values and score
sums (the casts and the two scalings are fully specified IEEE operations); end to end the scores
are held to 1e-4 of the float64 oracle."""
import ctypes
import logging

import numpy as np
import pytest
import torch

from oracle import score_oracle as so
from trak_amd import (
    BasicScoreComputer,
    ChunkedCudaProjector,
    CudaProjector,
    FeatureWriter,
    MmapSaver,
    ProjectionType,
    ScoreAccumulator,
    _lib,
    fast_jl,
)
from trak_amd.utils import gemm_nt, scores_finalize

pytestmark = pytest.mark.gpu


def reference_epilogue(projected, normalize_factor, dtype):
    """trak/traker.py:426-428 on a projection result."""
    g = projected.clone()
    g /= normalize_factor
    return g.to(dtype).cpu().clone().detach()


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("B,P,k", [(32, 5000, 1024), (5, 777, 512), (45, 3001, 512)])
def test_project_into_device_equals_reference_sequence(gpu, out_dtype, B, P, k):
    gen = torch.Generator().manual_seed(B + P)
    g = (torch.randn(B, P, generator=gen) * 3).half().to(gpu)
    nf = torch.sqrt(torch.tensor(float(P), dtype=torch.float32))
    want = reference_epilogue(fast_jl.project_rademacher_32(g, k, 11, 64), nf, out_dtype)
    out = torch.full((B, k), float("nan"), dtype=out_dtype, device=gpu)
    scale = float(torch.ones((), dtype=torch.float32) / nf)
    fast_jl.project_into(g, k, 11, 64, "rademacher", out, scale)
    assert torch.equal(out.cpu(), want)
    # wide range of magnitudes (fp16 subnormals and overflow to inf after the cast)
    big = (torch.randn(B, P, generator=gen) * 2000).half().to(gpu)
    want = reference_epilogue(fast_jl.project_rademacher_32(big, k, 3, 64), torch.tensor(1e-3), out_dtype)
    fast_jl.project_into(big, k, 3, 64, "rademacher", out, float(torch.ones(()) / torch.tensor(1e-3)))
    assert torch.equal(out.cpu(), want)
    tiny = (torch.randn(B, P, generator=gen) * 1e-3).half().to(gpu)
    want = reference_epilogue(fast_jl.project_rademacher_32(tiny, k, 3, 64), torch.tensor(3e3), out_dtype)
    fast_jl.project_into(tiny, k, 3, 64, "rademacher", out, float(torch.ones(()) / torch.tensor(3e3)))
    assert torch.equal(out.cpu(), want)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.float16])
def test_project_into_pinned_host_memory(gpu, out_dtype):
    B, P, k = 32, 40_000, 2048
    gen = torch.Generator().manual_seed(5)
    g = torch.randn(B, P, generator=gen).half().to(gpu)
    nf = torch.sqrt(torch.tensor(float(P)))
    want = reference_epilogue(fast_jl.project_normal_32(g, k, 2, 256), nf, out_dtype)
    wide = torch.zeros((B, 2 * k), dtype=out_dtype).pin_memory()
    out = wide[:, k // 2 : k // 2 + k]  # row pitch 2k, offset start
    fast_jl.project_into(g, k, 2, 256, "normal", out, float(torch.ones(()) / nf))
    torch.cuda.synchronize()
    assert torch.equal(out, want)
    assert float(wide[:, : k // 2].abs().sum()) == 0.0 and float(wide[:, k // 2 + k :].abs().sum()) == 0.0


def test_pageable_destination_is_refused_on_the_host(gpu):
    g = torch.randn(8, 1000).half().to(gpu)
    with pytest.raises(RuntimeError, match="page-locked"):
        fast_jl.project_into(g, 512, 0, 16, "rademacher", torch.zeros(8, 512), 1.0)
    with pytest.raises(RuntimeError):
        fast_jl.project_into(g, 512, 0, 16, "rademacher", torch.zeros(8, 256).pin_memory(), 1.0)
    # the C ABI itself asks HIP about the pointer and launches nothing
    lib = _lib.load()
    ws = torch.zeros(lib.trakhip_project_workspace(8, 1000, 512, 16), dtype=torch.uint8, device=gpu)
    pageable = np.zeros((8, 512), dtype=np.float32)
    rc = lib.trakhip_project_reduce_store(
        ctypes.c_void_p(ws.data_ptr()), 8, 1000, 512, 16, 1.0, _lib.F32,
        ctypes.c_void_p(pageable.ctypes.data), 512, None)
    assert rc == -11
    acc = torch.zeros(8, 512, device=gpu)
    rc = lib.trakhip_scores_finalize(
        ctypes.c_void_p(acc.data_ptr()), 512, 8, 512, 1.0, None, _lib.F32,
        ctypes.c_void_p(pageable.ctypes.data), 512, None)
    assert rc == -11
    torch.cuda.synchronize()
    assert float(fast_jl.project_rademacher_8(g, 512, 0, 16).abs().sum()) > 0  # the device is still fine


def _grad_dict(gen, B, device, dtype):
    shapes = {"conv.weight": (6, 3, 5, 5), "conv.bias": (6,), "fc.weight": (37, 123), "scalar": ()}
    return {k: torch.randn((B,) + s, generator=gen).to(dtype).to(device) for k, s in shapes.items()}


@pytest.mark.parametrize("store_dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("depth", [1, 2, 3])
def test_feature_writer_equals_reference_loop(gpu, store_dtype, depth):
    gen = torch.Generator().manual_seed(depth)
    k, N = 1024, 75
    batches = [_grad_dict(gen, b, gpu, torch.float16) for b in (32, 32, 11)]
    P = sum(v[0].numel() for v in batches[0].values())
    proj = CudaProjector(grad_dim=P, proj_dim=k, seed=4, proj_type=ProjectionType.rademacher, device=gpu,
                         max_batch_size=32)
    nf = torch.sqrt(torch.tensor(P, dtype=torch.float32))
    order = torch.randperm(N, generator=gen).numpy()
    inds = [order[:32], order[32:64], order[64:75]]
    npdt = np.float16 if store_dtype == torch.float16 else np.float32
    want = np.zeros((N, k), dtype=npdt)
    for grads, ind in zip(batches, inds):
        want[ind] = reference_epilogue(proj.project(grads, model_id=1), nf, store_dtype)
    got = np.zeros((N, k), dtype=npdt)
    writer = FeatureWriter(proj, k, nf, dtype=store_dtype, max_batch_size=32, depth=depth)
    for grads, ind in zip(batches, inds):
        writer.write(grads, 1, got, ind)
    writer.flush()
    assert np.array_equal(got.view(np.uint16 if npdt == np.float16 else np.uint32),
                          want.view(np.uint16 if npdt == np.float16 else np.uint32))
    # a dense [B, P] tensor takes the same path
    from trak_amd import vectorize

    got2 = np.zeros((N, k), dtype=npdt)
    for grads, ind in zip(batches, inds):
        writer.write(vectorize(grads, device=gpu), 1, got2, ind)
    writer.flush()
    assert np.array_equal(got2, want)
    with pytest.raises(ValueError):
        writer.write(torch.zeros(33, P, device=gpu, dtype=torch.float16), 1, got2, np.arange(33))


def test_feature_writer_with_a_projector_that_has_no_fused_path(gpu):
    gen = torch.Generator().manual_seed(9)
    k, B = 512, 16
    grads = _grad_dict(gen, B, gpu, torch.float16)
    sizes = [1 if v.dim() < 2 else v[0].numel() for v in grads.values()]
    # two chunks: (conv.weight, conv.bias) and (fc.weight, scalar)
    per = [sizes[0] + sizes[1], sizes[2] + sizes[3]]
    mk = lambda n, seed: CudaProjector(grad_dim=n, proj_dim=k, seed=seed, proj_type=ProjectionType.rademacher,
                                       device=gpu, max_batch_size=16)
    chunked = ChunkedCudaProjector([mk(per[0], 0), mk(per[1], 1)], max(per), per, B, gpu, torch.float16)
    nf = torch.sqrt(torch.tensor(float(sum(per))))
    want = reference_epilogue(chunked.project(grads, model_id=0), nf, torch.float16).numpy()
    got = np.zeros((B, k), dtype=np.float16)
    writer = FeatureWriter(chunked, k, nf, dtype=torch.float16, max_batch_size=B)
    writer.write(grads, 0, got, np.arange(B))
    writer.flush()
    assert np.array_equal(got, want)


def reference_finalize(acc_cpu, o2l_sum, n, np_dtype):
    """trak/traker.py:672-676."""
    out = np.zeros(acc_cpu.shape, dtype=np_dtype)
    out[:] = (acc_cpu.numpy() / n) * (o2l_sum / n)
    return out


@pytest.mark.parametrize("N,M", [(64, 128), (77, 37), (1, 1), (300, 6), (5, 1030)])
@pytest.mark.parametrize("half", [False, True])
def test_scores_finalize_equals_numpy_expression(gpu, N, M, half):
    gen = torch.Generator().manual_seed(N * M)
    acc = torch.randn(N, M, generator=gen) * 37.0
    npdt = np.float16 if half else np.float32
    o2l = (torch.rand(N, 1, generator=gen) * 3).numpy().astype(npdt)
    n = 3.0
    want = reference_finalize(acc, o2l, n, npdt)
    row = (o2l / n).astype(np.float32).reshape(-1)
    tdt = torch.float16 if half else torch.float32
    out = torch.zeros(N, M, dtype=tdt, device=gpu)
    scores_finalize(acc.to(gpu), n, torch.from_numpy(row), out)
    assert np.array_equal(out.cpu().numpy(), want)
    # strided source and page-locked, strided destination
    wide = torch.zeros(N, M + 9)
    wide[:, 3 : 3 + M] = acc
    host = torch.zeros(N, M + 5, dtype=tdt).pin_memory()
    scores_finalize(wide.to(gpu)[:, 3 : 3 + M], n, torch.from_numpy(row), host[:, 1 : 1 + M])
    torch.cuda.synchronize()
    assert np.array_equal(host[:, 1 : 1 + M].numpy(), want)
    assert float(host[:, 0].abs().sum()) == 0 and float(host[:, 1 + M :].abs().sum()) == 0


@pytest.mark.parametrize("half", [False, True])
def test_score_accumulator_equals_reference_loop(gpu, half):
    N, M, k, models = 210, 52, 512, 3
    gen = torch.Generator().manual_seed(17)
    dtype = torch.float16 if half else torch.float32
    npdt = np.float16 if half else np.float32
    sc = BasicScoreComputer(dtype=dtype, device=gpu)
    feats = [(torch.randn(N, k, generator=gen) / 8).to(dtype) for _ in range(models)]
    targs = [(torch.randn(M, k, generator=gen) / 8).to(dtype) for _ in range(models)]
    o2ls = [torch.rand(N, 1, generator=gen).numpy().astype(npdt) for _ in range(models)]
    # the reference's loop: CPU accumulator, numpy epilogue
    acc_cpu = torch.zeros(N, M)
    o2l_sum = np.zeros((N, 1), dtype=npdt)
    for f, t, o in zip(feats, targs, o2ls):
        sc.get_scores(f.to(gpu), t.to(gpu), accumulator=acc_cpu)
        o2l_sum += o
    want = reference_finalize(acc_cpu, o2l_sum, float(models), npdt)
    sa = ScoreAccumulator(sc, N, M, dtype=dtype)
    for f, t, o in zip(feats, targs, o2ls):
        sa.add(f.to(gpu), t.to(gpu), o)
    got = np.zeros((N, M), dtype=npdt)
    sa.finalize(got, chunk_bytes=M * got.itemsize * 64)  # four chunks through two staging buffers
    assert np.array_equal(got, want)
    got1 = np.zeros((N, M), dtype=npdt)
    sa.finalize(got1)  # one chunk
    assert np.array_equal(got1, want)
    dev = torch.zeros(N, M, dtype=dtype, device=gpu)
    sa.finalize(dev)
    assert np.array_equal(dev.cpu().numpy(), want)
    # and against the float64 oracle of the whole expression
    acc64 = sum(so.scores_f64(f.float().numpy(), t.float().numpy()) for f, t in zip(feats, targs))
    want64 = so.finalize_scores_f64(acc64, sum(o.astype(np.float64) for o in o2ls), models)
    tol = 2e-3 if half else 1e-4
    assert np.abs(got.astype(np.float64) - want64).max() <= tol * np.abs(want64).max()


def test_featurize_finalize_score_through_the_saver(gpu, tmp_path):
    """The whole path on one small problem: FeatureWriter -> MmapSaver stores -> BasicScoreComputer
    -> ScoreAccumulator -> scores store, against the float64 oracle fed with the same stored
    gradients (1e-4 relative)."""
    N, M, k = 768, 20, 512  # N > k keeps X^T X well conditioned
    gen = torch.Generator().manual_seed(23)
    saver = MmapSaver(save_dir=str(tmp_path), metadata={"JL dimension": k, "JL matrix type": "rademacher",
                                                        "train set size": N},
                      train_set_size=N, proj_dim=k, load_from_save_dir=True, logging_level=logging.ERROR,
                      use_half_precision=False)
    shapes_P = sum(int(np.prod(s)) if s else 1 for s in [(6, 3, 5, 5), (6,), (37, 123), ()])
    proj = CudaProjector(grad_dim=shapes_P, proj_dim=k, seed=0, proj_type=ProjectionType.rademacher, device=gpu,
                         max_batch_size=32)
    nf = torch.sqrt(torch.tensor(float(shapes_P)))
    sc = BasicScoreComputer(dtype=torch.float32, device=gpu, lambda_reg=1e-3)
    sa = ScoreAccumulator(sc, N, M)
    acc64 = np.zeros((N, M))
    o2l64 = np.zeros((N, 1))
    for model_id in (0, 1):
        saver.register_model_id(model_id, _allow_featurizing_already_registered=False)
        writer = FeatureWriter(proj, k, nf, dtype=torch.float32)
        for r0 in range(0, N, 32):
            inds = np.arange(r0, min(N, r0 + 32))
            writer.write(_grad_dict(gen, len(inds), gpu, torch.float16), model_id, saver.current_store["grads"], inds)
            saver.current_store["out_to_loss"][inds] = torch.rand(len(inds), 1, generator=gen).numpy()
            saver.current_store["is_featurized"][inds] = 1
        writer.flush()
        saver.serialize_current_model_id_metadata()
        assert saver.model_ids[model_id]["is_featurized"] == 1
        g = torch.as_tensor(np.asarray(saver.current_store["grads"]), device=gpu)
        feats = sc.get_x_xtx_inv(g, sc.get_xtx(g))
        saver.current_store["features"][:] = feats.cpu().numpy()
        saver.init_experiment("t", M, model_id)
        tw = FeatureWriter(proj, k, nf, dtype=torch.float32)
        tw.write(_grad_dict(gen, M, gpu, torch.float16), model_id, saver.current_store["t_grads"], np.arange(M))
        tw.flush()
        saver.load_current_store(model_id)
        sa.add(torch.as_tensor(np.asarray(saver.current_store["features"]), device=gpu),
               torch.as_tensor(np.asarray(saver.current_store["t_grads"]), device=gpu),
               np.asarray(saver.current_store["out_to_loss"]))
        X = np.asarray(saver.current_store["grads"], dtype=np.float64)
        f64 = so.x_xtx_inv_f64(X, so.xtx_f64(X), 1e-3)[0]
        acc64 += so.scores_f64(f64, np.asarray(saver.current_store["t_grads"], dtype=np.float64))
        o2l64 += np.asarray(saver.current_store["out_to_loss"], dtype=np.float64)
    saver.load_current_store(0, "t", M)
    sa.finalize(saver.current_store["t_scores"])
    saver.save_scores("t")
    want = so.finalize_scores_f64(acc64, o2l64, 2)
    got = np.load(tmp_path / "scores" / "t.mmap", mmap_mode="r")
    assert got.shape == (N, M)
    assert np.abs(np.asarray(got, dtype=np.float64) - want).max() <= 1e-4 * np.abs(want).max()


def test_projection_and_scoring_replay_from_a_hip_graph(gpu):
    """The library only launches kernels on the caller's stream (no allocation, no memset, no sync), so a
    caller can capture it: a captured projection + epilogue + score product is replayed three times
    with new inputs, with eager work and synchronizations in between, and must equal the eager
    result bit for bit every time."""
    B, P, k, M = 32, 30_000, 1024, 96
    gen = torch.Generator(device=gpu).manual_seed(5)
    g_static = torch.zeros(B, P, dtype=torch.float16, device=gpu)
    targets = torch.randn(M, k, generator=gen, device=gpu)
    feats = torch.empty(B, k, dtype=torch.float32, device=gpu)
    scores = torch.empty(B, M, device=gpu)
    from trak_amd.utils import split_rows

    def work():
        fast_jl.project_into(g_static, k, 3, 64, "rademacher", feats, 0.125)
        gemm_nt(feats, targets, out=scores)

    work()  # warm-up: sizes the cached workspace outside the capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            work()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        g_new = (torch.randn(B, P, generator=gen, device=gpu) * 0.01).half()
        g_static.copy_(g_new)
        graph.replay()
        torch.cuda.synchronize()
        got_feats, got_scores = feats.clone(), scores.clone()
        work()                                   # eager, same buffers
        torch.cuda.synchronize()
        assert torch.equal(got_feats, feats) and torch.equal(got_scores, scores), rep
        assert float(got_scores.abs().sum()) > 0
        _ = split_rows(targets)                  # unrelated eager work between replays


def test_gram_and_inverse_replay_from_a_hip_graph(gpu):
    """X^T X (operand split, k range shared out over three sets of workgroups, fixed-order combine) and the
    regularized inverse (about a hundred dependent launches, one of them heterogeneous) through the C
    ABI with caller-owned buffers: captured once, replayed with new inputs, equal to the eager result
    bit for bit, status word included."""
    lib = _lib.load()
    N, n, lam = 1500, 384, 1e-2
    gen = torch.Generator(device=gpu).manual_seed(9)
    x_static = torch.zeros(N, n, device=gpu)
    planes = torch.empty(lib.trakhip_split_bytes(n, N, _lib.F32), dtype=torch.uint8, device=gpu)
    gram_ws_bytes = lib.trakhip_gram_split_workspace(n, N, _lib.F32, 0)
    assert gram_ws_bytes == 3 * n * n * 4
    gram_ws = torch.empty(gram_ws_bytes, dtype=torch.uint8, device=gpu)
    xtx = torch.empty(n, n, device=gpu)
    inv = torch.empty(n, n, device=gpu)
    mean_abs = torch.zeros(1, device=gpu)
    status = torch.full((1,), -1, dtype=torch.int32, device=gpu)
    spd_ws = torch.empty(lib.trakhip_spd_inverse_workspace(n), dtype=torch.uint8, device=gpu)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())

    def work():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        assert lib.trakhip_split_rows(vp(x_static), _lib.F32, n, n, N, 1, vp(planes), planes.numel(), stream) == 0
        assert lib.trakhip_gram_split(vp(planes), n, N, _lib.F32, vp(xtx), n, 1.0, 0.0, vp(gram_ws), gram_ws_bytes,
                                      stream) == 0
        assert lib.trakhip_spd_inverse(vp(xtx), n, lam, vp(inv), n, n, 1, vp(mean_abs), vp(status), vp(spd_ws),
                                       spd_ws.numel(), stream) == 0

    x_static.copy_(torch.randn(N, n, generator=gen, device=gpu))
    work()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            work()
    torch.cuda.current_stream().wait_stream(side)
    for rep in range(3):
        x_static.copy_(torch.randn(N, n, generator=gen, device=gpu) * (1.0 + rep))
        status.fill_(-1)
        graph.replay()
        torch.cuda.synchronize()
        got = (xtx.clone(), inv.clone(), mean_abs.clone(), int(status.item()))
        status.fill_(-1)
        work()                                   # eager, same buffers
        torch.cuda.synchronize()
        assert got[3] == 0 and int(status.item()) == 0
        assert torch.equal(got[0], xtx) and torch.equal(got[1], inv) and torch.equal(got[2], mean_abs), rep
        a64 = x_static.double().T @ x_static.double() + lam * torch.eye(n, device=gpu, dtype=torch.float64)
        resid = a64 @ (got[1].double() * got[2].double()) - torch.eye(n, device=gpu, dtype=torch.float64)
        assert float(resid.abs().max()) < 1e-4
        _ = torch.randn(64, 64, device=gpu) @ torch.randn(64, 64, device=gpu)      # unrelated eager work
