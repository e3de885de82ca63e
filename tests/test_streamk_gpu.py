"""GPU parity tests of the dense stream-K GEMM, called through the C ABI
(streamk.gemm -> streamk_gemm_tn), against the CPU oracle f16_gemm_tn_ref on the
same seeded inputs.

Acceptance: exact equality where every sum is exactly representable; otherwise
max|C - C_ref| <= 2e-3 * max|C_ref| (fp32 accumulation on both sides, different
summation order, one fp16 rounding each) and the reference's own criterion,
cosine similarity >= 0.999 (include/reference.h:146-165).  Shapes follow the
reference's examples (gemm/readme.md:18-31)."""
import os
import sys

import numpy as np
import pytest

import _oracle as O

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "awesome-cute_amd"))

TOL = 2e-3


@pytest.fixture(scope="module")
def env():
    import torch
    import streamk
    assert torch.cuda.is_available()
    return torch, streamk


def inputs(m, n, k, seed, integers=False):
    rng = np.random.default_rng(seed)
    if integers:
        return (rng.integers(-3, 4, (m, k)).astype(np.float16),
                rng.integers(-3, 4, (n, k)).astype(np.float16))
    # the reference fills with uniform [-2, 2] (gemm_streamk.cu:33-36)
    return ((rng.random((m, k)) * 4 - 2).astype(np.float16),
            (rng.random((n, k)) * 4 - 2).astype(np.float16))


def gpu_gemm(env, A, B):
    torch, streamk = env
    dev = torch.device("cuda:0")
    print(f"  dense gemm M={A.shape[0]} N={B.shape[0]} K={A.shape[1]} "
          f"plan={streamk.plan(A.shape[0], B.shape[0], A.shape[1])[1]}", flush=True)
    C = streamk.gemm(torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev))
    torch.cuda.synchronize()
    return C.cpu().numpy()


def close(C, ref):
    C64, r64 = C.astype(np.float64), ref.astype(np.float64)
    assert np.isfinite(C64).all()
    assert np.abs(C64 - r64).max() <= TOL * np.abs(r64).max()
    cos = (C64 * r64).sum() / np.sqrt((C64 * C64).sum() * (r64 * r64).sum() + 1e-30)
    assert cos >= 0.999


# one tile; row tails; several tiles; stream-K tiles with 2, 3 and 4 slices on 256 CUs;
# 128 x 128 tiles (few tiles), 128 x 256 (640 x 7424) and 256 x 256 (1100 x 8192)
SHAPES = [(256, 256, 64), (1, 256, 64), (16, 256, 192), (255, 256, 128), (257, 512, 320),
          (300, 512, 1024), (256, 512, 4096), (700, 768, 1024), (512, 256, 2048),
          (1000, 2816, 512), (640, 7424, 512), (129, 256, 512), (200, 512, 768),
          (1024, 1024, 1024), (1100, 8192, 128)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_matches_oracle(env, m, n, k):
    A, B = inputs(m, n, k, m + n + k)
    close(gpu_gemm(env, A, B), O.dense_gemm_tn(A, B))


@pytest.mark.parametrize("m,n,k", [(256, 256, 64), (300, 512, 320), (256, 512, 2048), (700, 768, 512)])
def test_small_integers_are_exact(env, m, n, k):
    """Sums of products of integers in [-3, 3] stay below 2048 in magnitude for these
    depths only in the typical case, so compare through the oracle where the value is
    exactly representable and demand bit equality there."""
    A, B = inputs(m, n, k, 7, integers=True)
    want = A.astype(np.float64) @ B.astype(np.float64).T
    C = gpu_gemm(env, A, B).astype(np.float64)
    exact = np.abs(want) <= 2048
    assert exact.mean() > 0.99
    assert np.array_equal(C[exact], want[exact])


def test_one_hot_rows_return_rows_of_b(env):
    """A one-hot row of A selects a row of B^T: C[i, :] = B[:, k_i], bit for bit; this
    pins the operand layout for every k position of two stages and every column."""
    m, n, k = 128, 512, 128
    rng = np.random.default_rng(3)
    B = rng.standard_normal((n, k)).astype(np.float16)
    A = np.zeros((m, k), np.float16)
    A[np.arange(m), np.arange(m) % k] = 1
    C = gpu_gemm(env, A, B)
    assert np.array_equal(C.view(np.uint16), B[:, np.arange(m) % k].T.copy().view(np.uint16))


@pytest.mark.parametrize("m,n,k", [(4096, 4352, 4096), (1152, 4352, 4096), (4096, 4352, 10240),
                                   (4000, 4352, 512), (8100, 8192, 256), (2048, 2048, 2048),
                                   (1000, 4096, 4096)])
def test_reference_examples(env, m, n, k):
    """The reference's stream-K examples at full size (gemm/readme.md:27-31), and two
    shapes whose last row tile of 256 is partly empty: a sample of rows against the oracle, the whole result against torch's fp32 product by the
    reference's cosine criterion, and bit-identical results on a second run."""
    torch, streamk = env
    dev = torch.device("cuda:0")
    A, B = inputs(m, n, k, 11)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
    print(f"  dense gemm M={m} N={n} K={k} plan={streamk.plan(m, n, k)[1]}", flush=True)
    C = streamk.gemm(dA, dB)
    C2 = streamk.gemm(dA, dB)
    torch.cuda.synchronize()
    assert torch.equal(C, C2)
    rows = np.r_[0:4, 255:258, m - 3:m]
    close(C[torch.from_numpy(rows).to(dev)].cpu().numpy(), O.dense_gemm_tn(A[rows], B))
    ref = dA.float() @ dB.float().t()
    cos = torch.nn.functional.cosine_similarity(C.float().flatten(), ref.flatten(), dim=0).item()
    assert cos >= 0.999
    assert (C.float() - ref).abs().max().item() <= TOL * ref.abs().max().item()


def test_back_to_back_calls_share_the_scratch(env):
    """Stream-K launches one after the other on a stream reuse the partial-sum buffer and
    hand the tile counters back zeroed: a different problem in between must not disturb
    either result."""
    torch, streamk = env
    dev = torch.device("cuda:0")
    A1, B1 = inputs(700, 768, 1024, 1)
    A2, B2 = inputs(256, 512, 4096, 2)
    d = [torch.from_numpy(x).to(dev) for x in (A1, B1, A2, B2)]
    outs = []
    for _ in range(3):
        outs.append((streamk.gemm(d[0], d[1]), streamk.gemm(d[2], d[3])))
    torch.cuda.synchronize()
    for c1, c2 in outs[1:]:
        assert torch.equal(c1, outs[0][0]) and torch.equal(c2, outs[0][1])
    close(outs[0][0].cpu().numpy(), O.dense_gemm_tn(A1, B1))
    close(outs[0][1].cpu().numpy(), O.dense_gemm_tn(A2, B2))


def test_two_streams_run_side_by_side(env):
    """Stream-K launches on two streams at once: each stream has its own partial-sum
    buffer and tile counters; every result equals the one the same call gives alone."""
    torch, streamk = env
    dev = torch.device("cuda:0")
    A1, B1 = inputs(700, 768, 1024, 3)
    A2, B2 = inputs(256, 512, 4096, 4)
    d = [torch.from_numpy(x).to(dev) for x in (A1, B1, A2, B2)]
    alone = (streamk.gemm(d[0], d[1]), streamk.gemm(d[2], d[3]))
    torch.cuda.synchronize()
    outs = []
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    for _ in range(4):
        for st in streams:
            with torch.cuda.stream(st):
                outs.append((streamk.gemm(d[0], d[1]), streamk.gemm(d[2], d[3])))
    torch.cuda.synchronize()
    for c1, c2 in outs:
        assert torch.equal(c1, alone[0]) and torch.equal(c2, alone[1])


@pytest.mark.parametrize("m,n,k", [(700, 768, 1024), (512, 256, 2048), (2048, 2048, 512)])
def test_kernels_of_other_streams_beside_do_not_change_the_result(env, m, n, k):
    """A launch must give the same bits whatever else runs on the GPU.  Kernels of another
    stream that keep the compute units' LDS and memory busy (softmax, sort) stretch the
    latencies inside the GEMM; once, operand reads still in flight when the main loop ended
    landed in registers that already held the addresses of the partial sums."""
    torch, streamk = env
    dev = torch.device("cuda:0")
    A, B = inputs(m, n, k, 5)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
    alone = streamk.gemm(dA, dB)
    torch.cuda.synchronize()
    x = torch.randn(4096, 4096, device=dev)
    beside, main = torch.cuda.Stream(), torch.cuda.Stream()
    outs = []
    for it in range(30):
        with torch.cuda.stream(beside):
            if it % 2:
                torch.sort(x[:512], dim=1)
            else:
                for _ in range(3):
                    torch.softmax(x, dim=1)
        with torch.cuda.stream(main):
            outs.append(streamk.gemm(dA, dB))
    torch.cuda.synchronize()
    assert all(torch.equal(c, alone) for c in outs)
    close(alone.cpu().numpy(), O.dense_gemm_tn(A, B))


def test_degenerate_sizes_and_errors(env):
    torch, streamk = env
    dev = torch.device("cuda:0")
    C = torch.full((16, 256), 7.0, dtype=torch.half, device=dev)
    streamk.gemm(torch.zeros((16, 0), dtype=torch.half, device=dev),
                 torch.zeros((256, 0), dtype=torch.half, device=dev), C)
    torch.cuda.synchronize()
    assert not C.any().item()  # an empty sum
    assert streamk.gemm(torch.zeros((0, 64), dtype=torch.half, device=dev),
                        torch.zeros((256, 64), dtype=torch.half, device=dev)).shape == (0, 256)
    with pytest.raises(ValueError):
        streamk.gemm(torch.zeros((16, 64), dtype=torch.half, device=dev),
                     torch.zeros((128, 64), dtype=torch.half, device=dev))
    with pytest.raises(ValueError):
        streamk.gemm(torch.zeros((16, 32), dtype=torch.half, device=dev),
                     torch.zeros((256, 32), dtype=torch.half, device=dev))
    with pytest.raises(ValueError):
        streamk.gemm(torch.zeros((16, 64), dtype=torch.half, device=dev),
                     torch.zeros((256, 128), dtype=torch.half, device=dev))


def test_graph_replays_match_eager(env):
    """A captured stream-K launch replayed several times, with eager launches and
    synchronisations in between, gives the eager result every time (the tile counters
    are handed back zeroed by the kernel itself, nothing in the launch is a memset)."""
    torch, streamk = env
    dev = torch.device("cuda:0")
    A, B = inputs(700, 768, 1024, 5)
    dA, dB = torch.from_numpy(A).to(dev), torch.from_numpy(B).to(dev)
    A2, B2 = inputs(256, 512, 2048, 6)
    dA2, dB2 = torch.from_numpy(A2).to(dev), torch.from_numpy(B2).to(dev)
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        want = streamk.gemm(dA, dB).clone()      # also allocates this stream's scratch
        other = streamk.gemm(dA2, dB2).clone()
        side.synchronize()
        C = torch.zeros_like(want)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            streamk.gemm(dA, dB, C)
    for _ in range(4):
        C.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(C, want)
        with torch.cuda.stream(side):
            assert torch.equal(streamk.gemm(dA2, dB2), other)
            side.synchronize()


@pytest.mark.parametrize("tag", ["a", "b"])
def test_frozen_known_answers(env, tag):
    """The committed known answers (tests/golden/f16_gemm_known_answers.npz)."""
    z = np.load(os.path.join(ROOT, "tests", "golden", "f16_gemm_known_answers.npz"))
    A, B = z[f"{tag}_A"].view(np.float16), z[f"{tag}_B"].view(np.float16)
    close(gpu_gemm(env, A, B), z[f"{tag}_C"].view(np.float16))
