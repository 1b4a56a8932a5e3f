"""GPU parity tests of the JL projection: every call goes through the C ABI of libtrakhip.so
(via trak_amd.fast_jl / trak_amd.projectors) and is compared with the CPU oracle.

Tolerances (from the acceptance criteria of this build): matrix entries bit-exact; projected rows
within 1e-3 relative L2 for fp16/bf16 inputs and 1e-5 for fp32 inputs against a float64
contraction with the same matrix.
"""
import math

import numpy as np
import pytest
import torch

from oracle import jl_oracle as npo
from trak_amd import ChunkedCudaProjector, CudaProjector, ProjectionType, fast_jl

pytestmark = pytest.mark.gpu

R, G = npo.RADEMACHER, npo.NORMAL
NAMES = {R: "rademacher", G: "normal"}
TOL = {torch.float16: 1e-3, torch.bfloat16: 1e-3, torch.float32: 1e-5}


def fn(proj_type, n=32):
    return getattr(fast_jl, f"project_{NAMES[proj_type]}_{n}")


def rel_l2_rows(got, want):
    got = np.asarray(got, dtype=np.float64)
    want = np.asarray(want, dtype=np.float64)
    return np.linalg.norm(got - want, axis=1) / np.maximum(np.linalg.norm(want, axis=1), 1e-300)


def to_f32_numpy(t):
    return t.detach().float().cpu().numpy()


# ---- the matrix itself ------------------------------------------------------------------------


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize(
    "seed,tiles,P,f0,nf,c0,nc",
    [(0, 256, 1000, 0, 1000, 0, 8), (42, 256, 1_048_576, 4090, 300, 500, 12), (7, 108, 10_241, 9_900, 341, 2040, 8),
     (2**32 - 1, 256, 25, 0, 25, 0, 16), (7, 256, 11_689_512, 11_689_000, 512, 4064, 32)],
)
def test_device_matrix_is_bit_exact(gpu, c_oracle, proj_type, seed, tiles, P, f0, nf, c0, nc):
    got = fast_jl.materialize(seed, tiles, P, f0, nf, c0, nc, NAMES[proj_type], device=gpu).cpu().numpy()
    want = c_oracle.materialize(seed, tiles, P, f0, nf, c0, nc, proj_type)
    assert np.array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_one_hot_rows_read_the_matrix_back_exactly(gpu, c_oracle, proj_type, dtype):
    # project(e_f) = S[f, :] exactly: the MFMA path uses the same entries as the materializer
    P, k, tiles, seed = 5_000, 1024, 256, 17
    feats = [0, 1, 7, 8, 127, 128, 255, 256, 19, 20, 2559, 4096, 4998, 4999, 1234, 3333,
             39, 40, 41, 599, 600, 777, 2048, 2049, 3071, 3072, 4095, 4097, 4500, 4990, 4991, 4992]
    g = torch.zeros(32, P, dtype=dtype, device=gpu)
    for r, f in enumerate(feats):
        g[r, f] = 1.0
    out = fn(proj_type)(g, k, seed, tiles).cpu().numpy()
    for r, f in enumerate(feats):
        want = c_oracle.materialize(seed, tiles, P, f, 1, 0, k, proj_type)[0]
        assert np.array_equal(out[r], want), (r, f)


# ---- contraction parity against the float64 oracle --------------------------------------------


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize(
    "B,P,k,tiles",
    [(32, 20_000, 512, 256), (16, 10_002, 1024, 256), (9, 10_001, 512, 108), (1, 25, 512, 256), (45, 1049, 512, 256),
     (8, 70_001, 512, 7), (32, 9_000, 1536, 256), (12, 5_003, 2048, 64), (32, 6_001, 2560, 256),
     (64, 4_100, 1024, 16), (50, 3_001, 512, 5)],
)
def test_projection_matches_float64_contraction(gpu, c_oracle, proj_type, dtype, B, P, k, tiles):
    gen = torch.Generator(device="cpu").manual_seed(1000 + B + P)
    g = (torch.randn(B, P, generator=gen) * 1e-2).to(dtype).to(gpu)
    seed = 123 + B
    out = fn(proj_type)(g, k, seed, tiles)
    assert out.shape == (B, k) and out.dtype == torch.float32 and out.device == g.device  # fast_jl.cu:48-49,78
    # 512-, 1024- and 1536-column boundaries: a workgroup covers 512 columns when k is an odd multiple of
    # 512 (two column groups per wave), 1024 otherwise (four)
    cols = [c for c in (0, 31, 32, 511, 512, 1023, 1024, 1535, 2047, 2559) if c < k]
    g32 = to_f32_numpy(g)
    for c in cols:
        want = c_oracle.project(g32, seed, tiles, c, 1, proj_type)
        got = out[:, c : c + 1].cpu().numpy().astype(np.float64)
        err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
        assert err < TOL[dtype], (c, err)
    # and whole rows on a window of 64 columns
    want = c_oracle.project(g32, seed, tiles, k - 64, 64, proj_type)
    err = rel_l2_rows(out[:, k - 64 :].cpu().numpy(), want)
    assert err.max() < TOL[dtype], err.max()


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_tiny_values_and_exact_zeros(gpu, c_oracle, dtype):
    # gradient scales down to 1e-5 (fp16 subnormals) and 1 % exact zeros, as in the benchmark inputs
    B, P, k, tiles, seed = 32, 30_000, 512, 256, 7
    gen = torch.Generator(device="cpu").manual_seed(5)
    scale = 10 ** (torch.rand(P // 100, generator=gen) * 3 - 5)
    g = torch.randn(B, P, generator=gen) * scale.repeat_interleave(100)[None, :]
    g[torch.rand(B, P, generator=gen) < 0.01] = 0.0
    g = g.to(dtype).to(gpu)
    out = fn(R)(g, k, seed, tiles)
    want = c_oracle.project(to_f32_numpy(g), seed, tiles, 0, 64, R)
    assert rel_l2_rows(out[:, :64].cpu().numpy(), want).max() < TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("k,B", [(512, 23), (1024, 23), (512, 55), (1024, 64)])
def test_normal_projection_follows_the_rows_scale_from_chunk_to_chunk(gpu, c_oracle, dtype, k, B):
    # The normal kernel brings every 256-feature chunk of a row to fp16 with the row's own power of two
    # and carries the accumulators from one chunk's factor to the next.  Blocks of features whose sizes
    # differ by up to 2^±80 (far outside fp16), rows of different magnitude, all-zero stretches and
    # rows that are zero throughout must all come out as the float64 contraction says.
    # More than 32 rows of a 16-bit dtype go through the kernel 64 at a time (two 32-row blocks with their
    # own exponent lists); the special rows are repeated in the second block.
    P, tiles, seed = 9_000, 7, 31
    gen = torch.Generator(device="cpu").manual_seed(12)
    expo = torch.randint(-80, 81, (P // 300,), generator=gen).double()
    expo[::7] = 0
    scale = (2.0 ** expo).repeat_interleave(300)[None, :]
    g = (torch.randn(B, P, generator=gen).double() * scale)
    g *= (2.0 ** torch.randint(-20, 21, (B, 1), generator=gen).double())   # every row its own size
    g[:, 1200:2100] = 0.0           # an all-zero stretch longer than three chunks
    g[5] = 0.0                      # a row of zeros
    g[7, :] = 0.0
    g[7, 4321] = 3.0                # a one-hot row
    # one huge chunk followed by tiny ones, and the reverse: sums carried from a chunk of magnitude 2^90 must
    # not be blown up when chunks of magnitude 2^-90 follow, nor swamp a huge chunk that comes last
    g[9] = torch.randn(P, generator=gen).double() * 2.0 ** -90
    g[9, :256] = torch.randn(256, generator=gen).double() * 2.0 ** 90
    g[10] = torch.randn(P, generator=gen).double() * 2.0 ** -90
    g[10, P - 256 :] = torch.randn(256, generator=gen).double() * 2.0 ** 90
    if B > 50:
        g[37], g[41] = 0.0, g[9]
        g[39, :] = 0.0
        g[39, 8999] = -3.0
        g[50] = g[10]
    g = g.to(dtype)
    assert torch.isfinite(g).all()
    out = fn(G)(g.to(gpu), k, seed, tiles)
    assert torch.isfinite(out).all()
    want = c_oracle.project(to_f32_numpy(g), seed, tiles, k - 40, 40, G)
    got = out[:, k - 40 :].cpu().numpy().astype(np.float64)
    live = np.linalg.norm(want, axis=1) > 0
    assert not live[5] and not got[5].any()
    assert rel_l2_rows(got[live], want[live]).max() < TOL[dtype]
    # the one-hot row reads the matrix row back exactly (3 * entry is exact in fp32)
    s_row = c_oracle.materialize(seed, tiles, P, 4321, 1, 0, k, G)[0]
    assert np.array_equal(out[7].cpu().numpy(), 3.0 * s_row)
    if B > 50:
        assert not live[37] and not got[37].any()
        assert torch.equal(out[41], out[9]) and torch.equal(out[50], out[10])
        assert np.array_equal(out[39].cpu().numpy(), -3.0 * c_oracle.materialize(seed, tiles, P, 8999, 1, 0, k, G)[0])
        # a row's result does not depend on the rows it shares a pass with
        assert torch.equal(fn(G)(g[:32].to(gpu), k, seed, tiles), out[:32])
        assert torch.equal(fn(G)(g[32:].to(gpu), k, seed, tiles), out[32:])
    # scaling a row by a power of two scales its projection exactly
    g2 = g.clone()
    g2[3] *= 2.0 ** 9
    out2 = fn(G)(g2.to(gpu), k, seed, tiles)
    assert torch.equal(out2[3], out[3] * 2.0 ** 9)
    assert torch.equal(out2[4], out[4])


def test_row_pitch_and_unaligned_rows(gpu, c_oracle):
    # a column slice of a wider buffer (pitch > P) whose rows start at odd element offsets
    B, P, k, tiles, seed = 16, 3001, 512, 256, 3
    gen = torch.Generator(device="cpu").manual_seed(6)
    wide = torch.randn(B, 4099, generator=gen).half().to(gpu)
    view = wide[:, 77 : 77 + P]
    assert not view.is_contiguous()
    out = fn(R)(view, k, seed, tiles)
    out_c = fn(R)(view.contiguous(), k, seed, tiles)
    assert torch.equal(out, out_c)
    want = c_oracle.project(to_f32_numpy(view), seed, tiles, 100, 32, R)
    assert rel_l2_rows(out[:, 100:132].cpu().numpy(), want).max() < 1e-3


# ---- properties the reference's own tests assert ----------------------------------------------


@pytest.mark.parametrize("bs,input_size,output_size,seed", [(8, 1024, 512, 0), (8, 2048, 1024, 1), (8, 1024, 2048, 1)])
def test_shape(gpu, bs, input_size, output_size, seed):
    # tests/test_rademacher.py:21-39
    x = torch.ones((bs, input_size), dtype=torch.float16, device=gpu)
    num_sms = torch.cuda.get_device_properties(0).multi_processor_count
    assert fast_jl.project_rademacher_8(x, output_size, seed, num_sms).shape == (bs, output_size)


@pytest.mark.parametrize("P,seed,k,odd", [(10_240, 64, 1024, False), (10_241, 78, 2048, True)])
def test_even_odd(gpu, P, seed, k, odd):
    # tests/test_rademacher.py:65-108: all-ones input -> every output has the parity of P
    x = torch.ones((8, P), dtype=torch.float16, device=gpu)
    num_sms = torch.cuda.get_device_properties(0).multi_processor_count
    out = fast_jl.project_rademacher_8(x, k, seed, num_sms)
    assert torch.all(out % 2 == (1 if odd else 0))


def test_invalid_proj_dim_raises_value_error(gpu):
    # fast_jl/fast_jl_kernel.cuh:113-115 -> std::invalid_argument -> ValueError
    x = torch.ones((8, 1000), dtype=torch.float16, device=gpu)
    with pytest.raises(ValueError, match="multiple of 512"):
        fast_jl.project_rademacher_8(x, 1000, 0, 256)
    with pytest.raises(RuntimeError):
        fast_jl.project_rademacher_8(x.double(), 512, 0, 256)
    with pytest.raises(RuntimeError):
        fast_jl.project_rademacher_8(x[0], 512, 0, 256)


def _projector(P, k, seed, proj_type, dtype, **kw):
    return CudaProjector(grad_dim=P, proj_dim=k, seed=seed, proj_type=proj_type, device="cuda:0", dtype=dtype,
                         max_batch_size=32, **kw)


PROP = [
    (s, t, d, shape, k)
    for s in (0, 10**8)
    for t in (ProjectionType.normal, ProjectionType.rademacher)
    for d in (torch.float16, torch.float32)
    for shape, k in (((8, 10_000), 1024), ((9, 10_002), 1024), ((45, 1049), 1024), ((1, 25), 512))
]


@pytest.mark.parametrize("seed,proj_type,dtype,shape,k", PROP)
def test_seed_consistency(gpu, seed, proj_type, dtype, shape, k):
    # tests/test_jl.py:78-154: same seed -> same result, same instance and a new one
    g = torch.testing.make_tensor(*shape, device=gpu, dtype=dtype)
    p1 = _projector(shape[1], k, seed, proj_type, dtype)
    a = p1.project(g, model_id=0)
    assert torch.equal(a, p1.project(g, model_id=0))
    assert torch.equal(a, _projector(shape[1], k, seed, proj_type, dtype).project(g, model_id=0))
    # another model id or seed is another matrix (trak/projectors.py:409)
    assert not torch.equal(a, p1.project(g, model_id=1))
    assert not torch.equal(a, _projector(shape[1], k, seed + 1, proj_type, dtype).project(g, model_id=0))
    # model_id enters as seed + 10^4 * model_id
    assert torch.equal(p1.project(g, model_id=2), _projector(shape[1], k, seed + 20_000, proj_type, dtype).project(g, model_id=0))


@pytest.mark.parametrize("proj_type", [ProjectionType.normal, ProjectionType.rademacher])
@pytest.mark.parametrize("dtype", [torch.float16, torch.float32])
def test_norm_and_product_preservation(gpu, proj_type, dtype):
    # tests/test_jl.py:159-285 with the tests' own tolerances
    shape, k, seed = (16, 10_002), 4096, 1
    g = torch.testing.make_tensor(*shape, device=gpu, dtype=dtype)
    p = _projector(shape[1], k, seed, proj_type, dtype).project(g, model_id=0)
    rng = np.random.default_rng(0)
    delta = 0.05
    eps = np.sqrt(np.log(1 / delta) / k)
    ok = 0
    for _ in range(100):
        i, j = rng.choice(shape[0], size=2)
        n = (g[i].float() - g[j].float()).norm()
        pn = (p[i] - p[j]).norm() / np.sqrt(k)
        ok += int((n - pn).abs().item() <= 35 * eps * n.item())
    assert ok >= 100 * (1 - 3 * delta)
    # JL proper: squared norms within a few standard deviations (sqrt(2/k) relative)
    ratio = (p.norm(dim=1) ** 2 / k) / (g.float().norm(dim=1) ** 2)
    assert torch.all((ratio - 1).abs() < 6 * math.sqrt(2 / k))


@pytest.mark.parametrize("proj_type", [ProjectionType.normal, ProjectionType.rademacher])
def test_every_feature_contributes(gpu, proj_type):
    # tests/test_jl.py:290-389: single / first / last non-zero coordinate -> no output is zero
    B, P, k = 9, 10_002, 1024
    rng = np.random.default_rng(1)
    proj = _projector(P, k, 123, proj_type, torch.float32)
    for coords in ([0] * B, [P - 1] * B, rng.integers(0, P, size=B).tolist()):
        g = torch.zeros(B, P, device=gpu)
        for r, c in enumerate(coords):
            g[r, c] = 1.0 + r
        p = proj.project(g, model_id=0)
        assert (~torch.isclose(p, torch.zeros_like(p))).all().item()


@pytest.mark.parametrize("proj_type", [ProjectionType.normal, ProjectionType.rademacher])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_same_rows_same_features_through_chunks(gpu, proj_type, dtype):
    # tests/test_jl.py:394-446 and tests/test_jl_additional.py:63-87, on a forced 3-chunk split
    B, P, k = 8, 30_003, 512
    g = torch.testing.make_tensor(B, P, device=gpu, dtype=dtype)
    g[-1] = g[0]
    chunks = {i: x for i, x in enumerate(torch.chunk(g, 3, dim=1))}
    sizes = [v.size(1) for v in chunks.values()]
    seeds = np.random.default_rng(5).integers(low=0, high=500, size=3)   # trak/traker.py:294-296
    per_chunk = [_projector(sz, k, int(seeds[i]), proj_type, dtype) for i, sz in enumerate(sizes)]
    proj = ChunkedCudaProjector(per_chunk, max(sizes), sizes, B, "cuda:0", dtype)
    p = proj.project(chunks, model_id=0)
    assert p.shape == (B, k) and p.dtype == dtype               # trak/projectors.py:472-474
    assert torch.equal(p[0], p[-1])
    # the chunked result is the sum of the per-chunk projections (trak/projectors.py:490-514)
    want = sum(per_chunk[i].project(chunks[i].contiguous(), model_id=0) for i in range(3))
    assert torch.allclose(p.float(), want.to(dtype).float(), rtol=2e-2 if dtype != torch.float32 else 1e-6, atol=1e-2)
    proj.free_memory()


def test_orthogonality(gpu):
    # tests/test_jl.py:451-490
    B, P, k = 8, 10_000, 4096
    proj = _projector(P, k, 0, ProjectionType.rademacher, torch.float32)
    ok = 0
    for _ in range(10):
        g = torch.testing.make_tensor(B, P, device=gpu, dtype=torch.float32)
        g[-1] -= g[0] @ g[-1] / (g[0].norm() ** 2) * g[0]
        p = proj.project(g, model_id=0)
        ok += int(abs((p[0] @ p[-1]).item()) / k < 0.1 * (g[0].norm() * g[-1].norm()).item())
    assert ok > 3


def test_tile_count_changes_the_matrix_and_can_be_pinned(gpu):
    # the matrix depends on num_feature_tiles (fast_jl/random.cuh:15-17 with tile = blockIdx.y);
    # pinning num_sms reproduces another device's matrix (tests/test_jl_gpu_compatibility.py:59)
    g = torch.testing.make_tensor(8, 10_000, device=gpu, dtype=torch.float16)
    a = _projector(10_000, 512, 0, ProjectionType.rademacher, torch.float16, num_sms=108).project(g, 0)
    b = _projector(10_000, 512, 0, ProjectionType.rademacher, torch.float16, num_sms=108).project(g, 0)
    c = _projector(10_000, 512, 0, ProjectionType.rademacher, torch.float16).project(g, 0)
    assert torch.equal(a, b) and not torch.equal(a, c)
    assert torch.equal(a, fast_jl.project_rademacher_8(g, 512, 0, 108))


def test_dict_input_is_vectorized_in_dict_order(gpu):
    g = {"w": torch.randn(4, 3, 50, device=gpu), "b": torch.randn(4, device=gpu), "v": torch.randn(4, 70, device=gpu)}
    flat = torch.cat([g["w"].reshape(4, -1), g["b"].reshape(4, 1), g["v"]], dim=1)
    proj = _projector(flat.shape[1], 512, 9, ProjectionType.rademacher, torch.float32)
    assert torch.equal(proj.project(g, model_id=0), proj.project(flat, model_id=0))


# ---- full benchmark shape: size-independent properties and a column sample ---------------------


def test_full_size_resnet18_shape(gpu, c_oracle):
    B, P, k, seed = 32, 11_689_512, 4096, 7
    tiles = 256
    ones = torch.ones(B, P, dtype=torch.float16, device=gpu)
    out = fast_jl.project_rademacher_32(ones, k, seed, tiles)
    assert torch.all(out == out.round()) and torch.all(out % 2 == P % 2)      # parity closed form
    assert torch.all(out == out[0:1])                                          # equal rows
    # column sums of S are ~ N(0, P): the spread of the all-ones outputs must look like it
    z = out[0].double() / math.sqrt(P)
    assert abs(z.mean().item()) < 5 / math.sqrt(k) and abs(z.std().item() - 1) < 0.1
    del ones
    gen = torch.Generator(device="cpu").manual_seed(20_003)
    blocks = 62
    scale = 10 ** (torch.rand(blocks, generator=gen) * 3 - 5)
    edges = torch.linspace(0, P, blocks + 1).long()
    g = torch.randn(B, P, generator=gen)
    for i in range(blocks):
        g[:, edges[i] : edges[i + 1]] *= scale[i]
    g = g.half().to(gpu)
    out = fast_jl.project_rademacher_32(g, k, seed, tiles)
    # exact linearity under a power-of-two scale (fp16 * 2 is exact away from overflow)
    assert torch.equal(fast_jl.project_rademacher_32(g * 2, k, seed, tiles), out * 2)
    g32 = to_f32_numpy(g)
    for c in (0, 2049, 4095):
        want = c_oracle.project(g32, seed, tiles, c, 1, R)[:, 0]
        got = out[:, c].cpu().numpy().astype(np.float64)
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3


def test_full_size_resnet18_gradient_dict_through_the_projector(gpu, c_oracle):
    # what TRAKer.featurize hands to the projector at this shape: the dict of the 62 ResNet-18
    # parameter gradients (trak/gradient_computers.py:145-160), here with one log-uniform scale per
    # parameter.  CudaProjector.project(dict) reads it in place; the result must be the bits of
    # flatten-then-project and agree with the float64 contraction.
    import bench
    from trak_amd import vectorize

    shapes = bench.resnet18_param_shapes()
    B, k, seed = 32, 4096, 7
    P = sum(math.prod(sh) for sh in shapes)
    assert P == 11_689_512 and len(shapes) == 62
    gen = torch.Generator(device=gpu).manual_seed(20_003)
    scale = 10 ** (torch.rand(len(shapes), generator=gen, device=gpu) * 3 - 5)
    grads = {f"p{i}": (torch.randn(B, *sh, generator=gen, device=gpu) * scale[i]).half() for i, sh in enumerate(shapes)}
    proj = _projector(P, k, seed, ProjectionType.rademacher, torch.float16)
    out = proj.project(grads, model_id=0)
    flat = vectorize(grads, device=gpu)
    assert flat.shape == (B, P)
    dense = fast_jl.project_rademacher_32(flat, k, seed, proj.num_sms)
    assert torch.equal(out, dense)
    g32 = to_f32_numpy(flat)
    for c in (0, 1023, 1024, 3333, 4095):   # columns of all four column blocks, both ends
        want = c_oracle.project(g32, seed, proj.num_sms, c, 1, R)[:, 0]
        got = out[:, c].cpu().numpy().astype(np.float64)
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3, c
    # a second checkpoint (model_id) uses another matrix: seed + 10^4 * model_id (trak/projectors.py:409)
    out1 = proj.project(grads, model_id=1)
    assert torch.equal(out1, fast_jl.project_rademacher_32(flat, k, seed + 10_000, proj.num_sms))
    assert not torch.equal(out1, out)


def test_full_size_cpu_runnable_shape(gpu, c_oracle):
    # gradients [16, 1 048 576] fp32 iid N(0, 1e-3^2), k = 512, seed 42: every column against the
    # float64 contraction, to the fp32 bar
    B, P, k, seed, tiles = 16, 1_048_576, 512, 42, 256
    gen = torch.Generator(device="cpu").manual_seed(42)
    g = torch.randn(B, P, generator=gen) * 1e-3
    out = fast_jl.project_rademacher_16(g.to(gpu), k, seed, tiles).cpu().numpy()
    for c0 in (0, k - 48):
        want = c_oracle.project(g.numpy(), seed, tiles, c0, 48, R)
        assert rel_l2_rows(out[:, c0 : c0 + 48], want).max() < 1e-5
    # JL norm preservation at this shape: |Sg|^2 / k ~ |g|^2 within a few 1/sqrt(k)
    ratio = (out.astype(np.float64) ** 2).sum(1) / k / (g.double().numpy() ** 2).sum(1)
    assert np.abs(ratio - 1).max() < 6 * math.sqrt(2.0 / k)


def test_full_size_resnet9_shape(gpu, c_oracle):
    # gradients [32, 4 825 610] fp16 (P not a multiple of anything), N(0, 5e-4^2) with 1 % exact
    # zeros, k = 2048, seed 0, eight batches through one projector
    B, P, k, seed = 32, 4_825_610, 2048, 0
    proj = _projector(P, k, seed, ProjectionType.rademacher, torch.float16, num_sms=256)
    gen = torch.Generator(device=gpu).manual_seed(20_009)
    for batch in range(8):
        g = torch.randn(B, P, generator=gen, device=gpu) * 5e-4
        g[torch.rand(B, P, generator=gen, device=gpu) < 0.01] = 0.0
        g = g.half()
        assert 0.005 < float((g == 0).float().mean()) < 0.02
        out = proj.project(g, model_id=0)
        assert out.shape == (B, k) and out.dtype == torch.float32
        if batch in (0, 7):
            g32 = to_f32_numpy(g)
            for c in (0, 1023, 2047):
                want = c_oracle.project(g32, seed, 256, c, 1, R)[:, 0]
                got = out[:, c].cpu().numpy().astype(np.float64)
                assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3
        if batch == 0:
            first_in, first_out = g, out.clone()
    assert torch.equal(proj.project(first_in, model_id=0), first_out)  # no state between batches


def test_full_size_bert_normal_chunked_shape(gpu, c_oracle):
    # gradients [32, 109 482 240] bf16 in 4 parameter chunks, Student-t (nu = 3) * 1e-4, k = 4096,
    # seed 123, normal matrix, through ChunkedCudaProjector with TRAKer's per-chunk seeds
    # (trak/traker.py:290-310); two columns against the float64 contraction of every chunk
    B, P, k, seed, tiles = 32, 109_482_240, 4096, 123, 256
    sizes = [P // 4] * 4
    seeds = np.random.default_rng(seed).integers(low=0, high=500, size=4)
    per_chunk = [_projector(sz, k, int(seeds[i]), ProjectionType.normal, torch.bfloat16, num_sms=tiles)
                 for i, sz in enumerate(sizes)]
    proj = ChunkedCudaProjector(per_chunk, max(sizes), sizes, B, "cuda:0", torch.bfloat16)
    gen = torch.Generator(device=gpu).manual_seed(20_010)
    grads = {}
    for i, sz in enumerate(sizes):
        # Student-t with 3 degrees of freedom: normal / sqrt(chi2_3 / 3)
        z = torch.randn(B, sz, generator=gen, device=gpu)
        chi = sum(torch.randn(B, sz, generator=gen, device=gpu) ** 2 for _ in range(3)) / 3
        grads[f"chunk{i}"] = (z / chi.sqrt() * 1e-4).bfloat16()
        del z, chi
    out = proj.project(grads, model_id=0)
    assert out.shape == (B, k) and out.dtype == torch.bfloat16
    # the chunk projections in fp32, before the cast the chunked projector applies at the end
    parts = [per_chunk[i].project(grads[f"chunk{i}"], model_id=0) for i in range(4)]
    total = sum(p.double() for p in parts)
    assert torch.equal(total.float().bfloat16(), out) or (total.float() - out.float()).abs().max() <= \
        out.float().abs().max() * 2 ** -7
    for c in (5, 4090):
        want = np.zeros(B)
        for i in range(4):
            want += c_oracle.project(to_f32_numpy(grads[f"chunk{i}"]), int(seeds[i]), tiles, c, 1, G)[:, 0]
        got = total[:, c].cpu().numpy()
        assert np.linalg.norm(got - want) / np.linalg.norm(want) < 1e-3
    proj.free_memory()
    del grads
    torch.cuda.empty_cache()


# ---- the reference's uint32-overflow shapes (tests/test_jl.py:59-73, tests/test_jl_additional.py:11-44) ----


@pytest.mark.parametrize("shape", [(8, 180_645_096), (31, 180_645_096), (32, 180_645_096), (2, 780_645_096)])
def test_uint32_overflow_shapes_through_chunks(gpu, c_oracle, shape):
    # B * P >= 2^31 / 2^32: the reference's kernel indexes with uint32 `row * features`
    # (fast_jl/data_loading.cuh:37-41) and therefore chunks P; here addressing is 64-bit, and the
    # chunked path is exercised exactly as the reference's tests do.
    B, P = shape
    k, seed, dtype = 15_360, 123, torch.float32
    max_chunk_size = int(np.iinfo(np.uint32).max // B)
    num_chunks = int(np.ceil(P / max_chunk_size))
    g = torch.zeros(B, P, device=gpu, dtype=dtype)
    g[:, 0] = 1.0
    g[:, -1] = 2.0
    g[0, 12_345_678] = 3.0
    g[-1] = g[0]
    chunks = {i: x for i, x in enumerate(torch.chunk(g, num_chunks, dim=1))}
    sizes = [v.size(1) for v in chunks.values()]
    seeds = np.random.default_rng(seed).integers(low=0, high=500, size=len(chunks))
    per_chunk = [_projector(sz, k, int(seeds[i]), ProjectionType.rademacher, dtype) for i, sz in enumerate(sizes)]
    proj = ChunkedCudaProjector(per_chunk, max_chunk_size, sizes, B, "cuda:0", dtype)
    p = proj.project(chunks, model_id=0)
    assert p.shape == (B, k)
    assert torch.equal(p, proj.project(chunks, model_id=0))                  # seed consistency
    assert torch.equal(p[0], p[-1])                                          # same rows, same features
    # exact expectation from the oracle: row b = 1*S0[0,:] + 2*S_last[last,:] (+ 3*S[f,:] for rows 0 and B-1)
    tiles = per_chunk[0].num_sms
    first = c_oracle.materialize(int(seeds[0]), tiles, sizes[0], 0, 1, 0, k, R)[0]
    last = c_oracle.materialize(int(seeds[-1]), tiles, sizes[-1], sizes[-1] - 1, 1, 0, k, R)[0]
    ci, off = divmod(12_345_678, sizes[0]) if sizes[0] * (len(sizes) - 1) > 12_345_678 else (0, 12_345_678)
    mid = c_oracle.materialize(int(seeds[ci]), tiles, sizes[ci], off, 1, 0, k, R)[0]
    want_plain = first + 2.0 * last
    got = p.cpu().numpy()
    if B > 2:
        assert np.array_equal(got[1], want_plain)
    assert np.array_equal(got[0], want_plain + 3.0 * mid)
    proj.free_memory()
    del g, chunks
    torch.cuda.empty_cache()


# ---- gathered input: the gradient dict is projected in place -----------------------------------


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_gather_equals_vectorize_then_project(gpu, c_oracle, proj_type, dtype):
    from trak_amd import vectorize

    gen = torch.Generator(device="cpu").manual_seed(77)
    B = 19
    shapes = [(64, 3, 3, 3), (64,), (), (128, 64, 3, 3), (7,), (1,), (33, 5), (1000, 17), (2, 1, 1), (511,), (10, 10)]
    grads = {}
    for i, sh in enumerate(shapes):
        grads[f"p{i}"] = (torch.randn(B, *sh, generator=gen) * 1e-2).to(dtype).to(gpu)
    # one parameter arrives as a non-contiguous view (a column slice of a wider buffer)
    wide = (torch.randn(B, 300, generator=gen) * 1e-2).to(dtype).to(gpu)
    grads["view"] = wide[:, 10:210]
    flat = vectorize(grads, device=gpu)
    P, k, seed, tiles = flat.shape[1], 1024, 5, 256
    dense = fn(proj_type)(flat, k, seed, tiles)
    gathered = fast_jl.project_gather(list(grads.values()), k, seed, tiles, NAMES[proj_type])
    assert torch.equal(dense, gathered)
    # and against the oracle directly
    want = c_oracle.project(to_f32_numpy(flat), seed, tiles, 0, 32, proj_type)
    assert rel_l2_rows(gathered[:, :32].cpu().numpy(), want).max() < TOL[dtype]
    # the scale of the featurize epilogue (trak/traker.py:426) is applied in the reduction
    scaled = fast_jl.project_gather(list(grads.values()), k, seed, tiles, NAMES[proj_type], scale=1.0 / math.sqrt(P))
    assert torch.allclose(scaled, dense / math.sqrt(P), rtol=1e-6, atol=0)
    # CudaProjector takes the dict path
    proj = _projector(P, k, seed, ProjectionType(NAMES[proj_type]), dtype)
    assert torch.equal(proj.project(grads, model_id=0), dense)
    assert torch.equal(proj.project(flat, model_id=0), dense)


@pytest.mark.parametrize("B,k", [(45, 512), (70, 1024), (64, 2048)])
def test_gather_many_rows_and_tiny_segments(gpu, B, k):
    # B > 32: 16-bit gradients under a Rademacher matrix go through the kernel 64 rows at a time (two 32-row
    # blocks per generated operand); segments of one feature straddle every 16-byte piece
    from trak_amd import vectorize

    gen = torch.Generator(device="cpu").manual_seed(78)
    grads = {i: torch.randn(B, n, generator=gen).half().to(gpu) for i, n in enumerate([1, 1, 3, 1, 5, 2, 900, 1, 1, 7, 4000, 3])}
    flat = vectorize(grads, device=gpu)
    dense = fn(R)(flat, k, 11, 256)
    assert torch.equal(fast_jl.project_gather(list(grads.values()), k, 11, 256, "rademacher"), dense)
    # the same rows 32 at a time (the other kernel instance) give the same bits
    for b0 in range(0, B, 32):
        assert torch.equal(fn(R)(flat[b0:b0 + 32].contiguous(), k, 11, 256), dense[b0:b0 + 32])


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize("dtype,B", [(torch.float16, 32), (torch.bfloat16, 64), (torch.float16, 40)])
def test_gather_long_tiles_and_segment_boundaries(gpu, proj_type, dtype, B):
    # Few feature tiles, so that most chunks lie wholly inside a tile and inside one tensor (they are loaded like
    # the chunks of a dense matrix, from the segment the workgroup keeps in scalar registers), with tensor
    # boundaries on and off multiples of 256 features, tensors shorter than a chunk in between, row pitches
    # larger than the tensor (column slices) and a last tensor that ends inside a chunk.
    from trak_amd import vectorize

    gen = torch.Generator(device="cpu").manual_seed(79)
    sizes = [256 * 40, 256 * 3, 5, 256 * 17 + 1, 255, 256 * 60 - 6, 1, 256 * 25, 31_003, 256, 256 * 9 + 130]
    grads = []
    for i, n in enumerate(sizes):
        if i % 3 == 1:   # a column slice of a wider buffer: row pitch > n, rows not 16-byte aligned
            wide = (torch.randn(B, n + 37, generator=gen) * 1e-2).to(dtype).to(gpu)
            grads.append(wide[:, 5:5 + n])
        else:
            grads.append((torch.randn(B, n, generator=gen) * 1e-2).to(dtype).to(gpu))
    flat = vectorize({i: g for i, g in enumerate(grads)}, device=gpu)
    for tiles, k in ((7, 1024), (1, 512), (64, 2048)):
        dense = fn(proj_type)(flat, k, 21, tiles)
        gathered = fast_jl.project_gather(grads, k, 21, tiles, NAMES[proj_type])
        assert torch.equal(dense, gathered), (tiles, k)


# ---- more than 32 rows: the batch is walked 64 or 32 rows at a time -----------------------------


@pytest.mark.parametrize("proj_type", [R, G])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("B", [33, 64, 100, 129])
def test_many_rows(gpu, c_oracle, proj_type, dtype, B):
    P, k, tiles, seed = 9_001, 512, 256, 21
    gen = torch.Generator(device="cpu").manual_seed(B)
    g = (torch.randn(B, P, generator=gen) * 1e-2).to(dtype).to(gpu)
    out = fn(proj_type)(g, k, seed, tiles)
    assert out.shape == (B, k)
    want = c_oracle.project(to_f32_numpy(g), seed, tiles, 480, 32, proj_type)
    assert rel_l2_rows(out[:, 480:].cpu().numpy(), want).max() < TOL[dtype]
    # every row is projected by the same matrix whichever pass it falls into: one-hot rows read it back
    e = torch.zeros(B, P, dtype=dtype, device=gpu)
    feats = [(37 * r) % P for r in range(B)]
    e[torch.arange(B), torch.tensor(feats)] = 1.0
    got = fn(proj_type)(e, k, seed, tiles).cpu().numpy()
    for r in (0, 31, 32, 33, 63, B - 1):
        if r < B:
            assert np.array_equal(got[r], c_oracle.materialize(seed, tiles, P, feats[r], 1, 0, k, proj_type)[0]), r
    # a batch and its first 32 rows agree
    head = fn(proj_type)(g[:32].contiguous(), k, seed, tiles)
    assert torch.equal(out[:32], head)   # same launch shape, same matrix, same order of additions


def test_many_rows_gather(gpu):
    from trak_amd import vectorize

    gen = torch.Generator(device="cpu").manual_seed(5)
    grads = {i: torch.randn(100, n, generator=gen).half().to(gpu) for i, n in enumerate([300, 1, 4097, 15, 2000])}
    flat = vectorize(grads, device=gpu)
    assert torch.equal(fast_jl.project_gather(list(grads.values()), 512, 3, 256, "rademacher"), fn(R)(flat, 512, 3, 256))


def test_workspace_cache_is_bounded_and_streams_do_not_share_scratch(gpu):
    # one scratch buffer per (device, stream), at most eight of them kept; a projection on a side stream gives
    # the bits of one on the default stream
    g = (torch.randn(8, 3_000, generator=torch.Generator().manual_seed(4)) * 1e-2).half().to(gpu)
    want = fn(R)(g, 512, 3, 256)
    torch.cuda.synchronize()
    fast_jl.free_workspaces()
    streams = [torch.cuda.Stream(device=gpu) for _ in range(11)]
    for s in streams:
        with torch.cuda.stream(s):
            got = fn(R)(g, 512, 3, 256)
        s.synchronize()
        assert torch.equal(got, want)
    assert 1 <= len(fast_jl._workspaces) <= fast_jl._WORKSPACE_CACHE
    kept = {key[1] for key in fast_jl._workspaces}
    assert streams[-1].cuda_stream in kept and streams[0].cuda_stream not in kept   # least recently used went first
    fast_jl.free_workspaces()
    assert not fast_jl._workspaces and not fast_jl._segment_tables
