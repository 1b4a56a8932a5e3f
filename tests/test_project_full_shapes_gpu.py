"""Bit-exactness of the projection kernels at the benchmark shapes, through the C ABI.

A gradient row that is 1.0 at one feature and zero elsewhere projects to row f of the matrix, exactly:
every one of the proj_dim outputs is compared with the CPU oracle's entry, so a wrong block index, tile,
column or bit anywhere on the path (the run of chunks a workgroup walks, the hand-over from one run to the
next, the column blocks and the waves' column groups, the XCD placement) shows as a mismatch.  The features are
the ones where the bookkeeping changes: both ends of the gradient, both sides of tile boundaries, the partial
last chunk of a tile, both sides of every kind of run boundary (at a tile start and inside a tile), both lane
halves and the first / last MFMA step of a chunk.  Mirrors the reference's coordinate tests
(tests/test_jl.py:290-389) at full size.
"""
import math

import numpy as np
import pytest
import torch

from oracle import jl_oracle as npo
from trak_amd import CudaProjector, ProjectionType, fast_jl

pytestmark = pytest.mark.gpu

R, G = npo.RADEMACHER, npo.NORMAL
NAMES = {R: "rademacher", G: "normal"}
CHUNK = 256


def launch_plan(P, k, tiles, cus):
    """The split of a launch as the library documents it: feature tiles of ceil(P / T) features walked in
    chunks of 256, column blocks of 1024 columns (768 or 512 when k is an odd multiple of 512), and
    floor(CUs / column blocks) runs of consecutive chunks."""
    T = min(P, tiles)
    fts = (P - 1) // T + 1
    cpt = (fts + CHUNK - 1) // CHUNK
    total = T * cpt
    col_blocks = k // 1024 if k % 1024 == 0 else k // 768 if k % 768 == 0 else k // 512
    groups = max(1, min(total, cus // col_blocks))
    cpg = (total + groups - 1) // groups
    groups = (total + cpg - 1) // cpg
    return T, fts, cpt, cpg, groups


def interesting_features(P, k, tiles, cus, limit):
    T, fts, cpt, cpg, groups = launch_plan(P, k, tiles, cus)
    feats = [0, 1, 7, 8, 127, 128, 255, 256, P - 1, P - 2, P - 9, P - 129, P - 257]
    # tile boundaries, and the partial last chunk of a tile
    for t in (1, 2, T // 2, T - 1):
        lo = t * fts
        feats += [lo - 1, lo, lo + 127, lo + 128, lo - (fts % CHUNK or CHUNK), lo - (fts % CHUNK or CHUNK) - 1]
    # both sides of run boundaries: first chunk of run g starts at chunk g * cpg of the flattened (tile, chunk) list
    inside = at_start = 0
    for g in range(1, groups):
        c = g * cpg
        t, s = divmod(c, cpt)
        f = t * fts + s * CHUNK
        if f >= P:
            continue
        kind_inside = s != 0
        if (kind_inside and inside < 6) or (not kind_inside and at_start < 4) or g in (groups - 1, groups // 2):
            # last feature of the previous run (the end of the previous tile when the run starts a tile)
            feats += [f - 1, f, f + 255, min(f + 256, P - 1)]
            inside += kind_inside
            at_start += not kind_inside
    feats = [f for f in dict.fromkeys(feats) if 0 <= f < P]
    return feats[:limit]


def check_rows(out, feats, oracle, seed, tiles, P, k, proj_type, tag):
    got = out.cpu().numpy()
    for r, f in enumerate(feats):
        want = oracle.materialize(seed, tiles, P, f, 1, 0, k, proj_type)[0]
        assert np.array_equal(got[r].view(np.uint32), want.view(np.uint32)), (tag, r, f, int((got[r] != want).sum()))


def one_hot(B, P, feats, dtype, gpu):
    g = torch.zeros(B, P, dtype=dtype, device=gpu)
    idx = torch.tensor(feats[:B], device=gpu)
    g[torch.arange(len(idx), device=gpu), idx] = 1.0
    return g


CASES = [
    # name, rows per call, P, k, seed, dtype, matrix type
    ("resnet18", 32, 11_689_512, 4096, 7, torch.float16, R),
    ("resnet18_64rows", 64, 11_689_512, 4096, 7, torch.float16, R),
    ("resnet9", 32, 4_825_610, 2048, 0, torch.float16, R),
    ("resnet18_k3072", 32, 11_689_512, 3072, 7, torch.float16, R),     # runs that start inside a tile
    ("resnet18_k15360", 32, 11_689_512, 15_360, 7, torch.float16, R),  # 15 column blocks, 17 runs
    ("resnet18_k1536", 32, 11_689_512, 1536, 7, torch.bfloat16, R),    # 768-column workgroups
    ("resnet18_k2560", 32, 11_689_512, 2560, 7, torch.float16, R),     # 512-column workgroups
    ("resnet18_k1536_normal_64rows", 64, 11_689_512, 1536, 7, torch.float16, G),
    ("bert_chunk_normal", 32, 27_370_560, 4096, 123, torch.bfloat16, G),
    ("bert_chunk_normal_64rows", 64, 27_370_560, 4096, 123, torch.bfloat16, G),
]


@pytest.mark.parametrize("name,B,P,k,seed,dtype,proj_type", CASES, ids=[c[0] for c in CASES])
def test_one_hot_rows_at_benchmark_shapes(gpu, c_oracle, name, B, P, k, seed, dtype, proj_type):
    tiles = cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    feats = interesting_features(P, k, tiles, cus, limit=64)
    assert len(feats) >= 40, len(feats)
    project = getattr(fast_jl, f"project_{NAMES[proj_type]}_32")
    g = torch.zeros(B, P, dtype=dtype, device=gpu)
    rows = torch.arange(B, device=gpu)
    for i in range(0, len(feats), B):
        part = feats[i:i + B]
        idx = torch.tensor(part, device=gpu)
        g[rows[:len(part)], idx] = 1.0
        out = project(g, k, seed, tiles)
        check_rows(out, part, c_oracle, seed, tiles, P, k, proj_type, name)
        assert not out[len(part):].any()       # rows that are all zero stay zero
        g[rows[:len(part)], idx] = 0.0


def test_one_hot_rows_through_the_resnet18_gradient_dict(gpu, c_oracle):
    # the gathered kernel at the headline shape: features at both ends of parameter tensors as well
    import bench

    shapes = bench.resnet18_param_shapes()
    B, k, seed = 32, 4096, 7
    sizes = [math.prod(sh) for sh in shapes]
    P = sum(sizes)
    tiles = cus = torch.cuda.get_device_properties(gpu).multi_processor_count
    firsts = np.concatenate([[0], np.cumsum(sizes)])[:-1].tolist()
    feats = interesting_features(P, k, tiles, cus, limit=40)
    for i in (1, 2, 3, 20, 40, 60, 61):      # first and last feature of some tensors (the three 64-element ones too)
        feats += [firsts[i], firsts[i] + sizes[i] - 1]
    feats = list(dict.fromkeys(feats))[:64]
    grads = {f"p{i}": torch.zeros(B, *sh, dtype=torch.float16, device=gpu) for i, sh in enumerate(shapes)}
    flats = [g.view(B, -1) for g in grads.values()]
    proj = CudaProjector(P, k, seed, ProjectionType.rademacher, gpu, 32)

    def put(f, r, value):
        i = int(np.searchsorted(firsts, f, side="right") - 1)
        flats[i][r, f - firsts[i]] = value

    for i0 in range(0, len(feats), B):
        part = feats[i0:i0 + B]
        for r, f in enumerate(part):
            put(f, r, 1.0)
        out = proj.project(grads, model_id=0)
        check_rows(out, part, c_oracle, seed, tiles, P, k, R, "resnet18_dict")
        for r, f in enumerate(part):
            put(f, r, 0.0)


def test_float64_contraction_on_every_column_slot_of_the_headline_shape(gpu, c_oracle):
    # one column for every (column block, wave, column group of the wave) of the launch, 128 in all, with the
    # lane varied as well; four gradient rows against the float64 contraction (all rows: test_project_gpu.py)
    B, P, k, seed, tiles = 32, 11_689_512, 4096, 7, 256
    gen = torch.Generator(device=gpu).manual_seed(20_011)
    scale = 10 ** (torch.rand(62, generator=gen, device=gpu) * 3 - 5)
    g = torch.randn(B, P, generator=gen, device=gpu)
    edges = torch.linspace(0, P, 63).long().tolist()
    for i in range(62):
        g[:, edges[i]:edges[i + 1]] *= scale[i]
    g = g.half()
    out = fast_jl.project_rademacher_32(g, k, seed, tiles).cpu().numpy().astype(np.float64)
    rows = [0, 13, 20, 31]
    g32 = g[rows].float().cpu().numpy()
    worst = 0.0
    for slot in range(128):
        c = 32 * slot + (7 * slot + 3) % 32
        want = c_oracle.project(g32, seed, tiles, c, 1, R)[:, 0]
        got = out[rows, c]
        worst = max(worst, float(np.abs(got - want).max() / np.abs(want).max()))
    assert worst < 1e-3, worst


# ---- the reference's largest shapes (tests/test_rademacher_additional.py:18-60, tests/test_jl.py:66-69) ----


@pytest.mark.parametrize("bs", [8, 48])
@pytest.mark.parametrize("k", [2048, 15_360])
def test_all_ones_parity_form_at_180m_features(gpu, c_oracle, bs, k):
    # all-ones input: every output is a sum of P values +-1, i.e. an integer of P's parity
    # (tests/test_rademacher.py:65-108), equal for all rows, and S's column sums are ~ N(0, P); beyond
    # 2^24 such sums would stop being exact in fp32 - here |sum| stays far below
    P, seed = 180_645_096, 0
    tiles = torch.cuda.get_device_properties(gpu).multi_processor_count
    ones = torch.ones(bs, P, dtype=torch.float16, device=gpu)
    out = fast_jl.project_rademacher_8(ones, k, seed, tiles)
    assert out.shape == (bs, k)
    assert torch.all(out == out.round()) and torch.all(out % 2 == P % 2)
    assert torch.all(out == out[0:1])
    z = out[0].double() / math.sqrt(P)
    assert abs(z.mean().item()) < 5 / math.sqrt(k) and abs(z.std().item() - 1) < 0.1
    # three columns against the oracle's exact column sums (computed from one all-ones row)
    row = np.ones((1, P), dtype=np.float32)
    for c in (0, k // 2 + 1, k - 1):
        want = c_oracle.project(row, seed, tiles, c, 1, R)[0, 0]
        assert float(out[0, c]) == want, (c, float(out[0, c]), want)
    del ones
    torch.cuda.empty_cache()
