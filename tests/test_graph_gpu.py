"""The library's launches under HIP graph capture: every entry point is kernels only (no
allocation, no memset, no synchronisation), so a caller may record a step once and replay it.
Each case records its calls into a graph on static buffers, then replays it several times with
new inputs copied in and the program's own eager work and synchronisations between the replays,
and checks every replay against the same calls made eagerly."""
import pytest
import torch

from genbmm_amd import _lib

pytestmark = pytest.mark.gpu
P = _lib.ptr


def replay_and_compare(gpu, make_inputs, statics, outputs, step):
    """step(): the library calls on the static tensors.  Records it, then three replays on fresh
    inputs, each compared with an eager run of the same step on the same inputs."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):           # warm-up outside the capture (first-call set-up)
        step()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        step()
    for rep in range(3):
        fresh = make_inputs(rep)
        for dst, src in zip(statics, fresh):
            dst.copy_(src)
        for o in outputs:
            o.fill_(float("nan")) if o.is_floating_point() else o.fill_(-7)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outputs]
        # eager work of the program's own between the replays
        for o in outputs:
            o.fill_(float("nan")) if o.is_floating_point() else o.fill_(-7)
        step()
        torch.cuda.synchronize()
        for g, o in zip(got, outputs):
            assert torch.equal(g, o), rep


@pytest.mark.parametrize("B,M,K,N", [(6, 256, 128, 256), (40, 64, 64, 64), (5, 128, 100, 96), (2, 96, 4096, 96)])
def test_logbmm_step_replays(gpu, B, M, K, N):
    """Forward and backward on the caller's workspace: matrix-core tiles, whole-item kernels,
    one tile per item, and a forward that cuts its reduction into pieces."""
    lib = _lib.load()
    a, b, g = (torch.empty(*s, device=gpu) for s in ((B, M, K), (B, K, N), (B, M, N)))
    out, ga, gb = torch.empty(B, M, N, device=gpu), torch.empty_like(a), torch.empty_like(b)
    stats = torch.empty(lib.genbmm_logbmm_stats_size(B, M, K, N), device=gpu)

    def make(rep):
        torch.manual_seed(100 + rep)
        x, y, z = torch.randn(B, M, K, device=gpu), torch.randn(B, K, N, device=gpu), torch.randn(B, M, N, device=gpu)
        if rep == 1:
            x[0, ::2, 0] += 150.0     # tiles that need the exact fix-up
            y[0, 0, :] -= 150.0
        return x, y, z

    def step():
        s = _lib.stream_of(a)
        assert lib.genbmm_logbmm_fwd(P(a), P(b), P(out), P(stats), B, M, K, N, s) == 0
        assert lib.genbmm_logbmm_bwd(P(a), P(b), P(out), P(g), P(stats), P(ga), P(gb), B, M, K, N, s) == 0

    for t, src in zip((a, b, g), make(9)):
        t.copy_(src)
    replay_and_compare(gpu, make, (a, b, g), (out, ga, gb), step)


@pytest.mark.parametrize("B,M,K,N", [(3, 130, 97, 200), (2, 64, 4096, 64)])
def test_max_and_sample_steps_replay(gpu, B, M, K, N):
    """maxbmm (also the shape whose reduction the library cuts into pieces: its atomics start
    from cells that an initialising kernel, not a memset, has filled), its backward, and samplebmm."""
    lib = _lib.load()
    a, b, g = (torch.empty(*s, device=gpu) for s in ((B, M, K), (B, K, N), (B, M, N)))
    out, so = torch.empty(B, M, N, device=gpu), torch.empty(B, M, N, device=gpu)
    idx, sidx = (torch.empty(B, M, N, dtype=torch.int32, device=gpu) for _ in range(2))
    ga, gb = torch.empty_like(a), torch.empty_like(b)
    stats = torch.empty(lib.genbmm_samplebmm_stats_size(B, M, K, N), device=gpu)

    def make(rep):
        torch.manual_seed(200 + rep)
        r = lambda *s: torch.round(torch.randn(*s, device=gpu) * 4) / 4
        return r(B, M, K), r(B, K, N), r(B, M, N)

    def step():
        s = _lib.stream_of(a)
        assert lib.genbmm_maxbmm_fwd(P(a), P(b), P(out), P(idx), B, M, K, N, s) == 0
        assert lib.genbmm_argmax_bwd(P(idx), P(g), P(ga), P(gb), B, M, K, N, s) == 0
        assert lib.genbmm_samplebmm_fwd(P(a), P(b), P(so), P(sidx), P(stats), 11, 3, B, M, K, N, s) == 0

    for t, src in zip((a, b, g), make(9)):
        t.copy_(src)
    replay_and_compare(gpu, make, (a, b, g), (out, idx, ga, gb, so, sidx), step)


def test_banded_step_replays(gpu):
    """Banded log product on its workspace and its backward, 65 diagonals per operand (the
    block kernel on the bf16 matrix instruction) and 9 (the memory-fed kernels)."""
    lib = _lib.load()
    for lu, n, B in ((32, 300, 3), (4, 200, 5)):
        W = 2 * lu + 1
        Wo = 2 * W - 1
        a, b, g = torch.empty(B, n, W, device=gpu), torch.empty(B, n, W, device=gpu), torch.empty(B, n, Wo, device=gpu)
        out, ga, gb = torch.empty(B, n, Wo, device=gpu), torch.empty_like(a), torch.empty_like(b)
        ws = torch.empty(lib.genbmm_banded_workspace_size(lu, lu, lu, lu, B, n), device=gpu)

        def make(rep):
            torch.manual_seed(300 + rep)
            return torch.randn(B, n, W, device=gpu), torch.randn(B, n, W, device=gpu), torch.randn(B, n, Wo, device=gpu)

        def step():
            s = _lib.stream_of(a)
            assert lib.genbmm_banded_fwd(P(a), lu, lu, P(b), lu, lu, P(out), None, P(ws), B, n, 0, s) == 0
            assert lib.genbmm_banded_bwd(P(a), lu, lu, P(b), lu, lu, P(out), None, P(ws), P(g), P(ga), P(gb), B, n, 0, s) == 0

        for t, src in zip((a, b, g), make(9)):
            t.copy_(src)
        replay_and_compare(gpu, make, (a, b, g), (out, ga, gb), step)
