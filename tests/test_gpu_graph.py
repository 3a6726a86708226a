"""moe_forward is enqueue-only with fixed scratch addresses: it can be captured into a HIP graph
(the reference captures its decode step, src/gpu/parts/40_model.inc:8011-8016).  The graph is
replayed several times with eager calls and synchronisations in between; every replay must
reproduce the eager result bit for bit (same kernels, same order)."""
import numpy as np
import pytest

from helpers import HostLayer

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("fmt,T", [("q4cp", 1), ("q4cp", 7), ("q4cp", 20), ("q4cp", 48), ("q4k", 1), ("q4k", 9)])
def test_forward_under_graph_capture(oracle, fmt, T):
    import torch
    rng = np.random.default_rng(5 + T)
    d, mid, E, k = 1024, 256, 16, 4
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt)
    m, dev = hl.to_gpu(max_tokens=64)
    xs = [torch.from_numpy(rng.standard_normal((T, d), dtype=np.float32)).cuda() for _ in range(3)]
    x = torch.empty((T, d), dtype=torch.float32, device="cuda")
    y = torch.empty((T, d), dtype=torch.float32, device="cuda")
    eager = []
    for xi in xs:  # eager results (also the warm-up that one-time kernel attributes need)
        x.copy_(xi)
        m.forward(0, x, y)
        eager.append(y.clone())
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    x.copy_(xs[0])
    with torch.cuda.graph(g):
        m.forward(0, x, y)
    for rep in range(3):
        for i, xi in enumerate(xs):
            x.copy_(xi)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager[i]), (rep, i)
            # eager work between replays
            y.zero_()
            m.forward(0, xs[(i + 1) % 3], y)
            torch.cuda.synchronize()
            assert torch.equal(y, eager[(i + 1) % 3])
    m.close()


@pytest.mark.parametrize("variant,T", [("table", 1), ("table", 4), ("table", 9), ("table", 48), ("dense", 1), ("dense", 6),
                                       ("dense", 48), ("ggmix", 3), ("ggmix", 48)])
def test_other_paths_under_graph_capture(oracle, variant, T):
    """The same for the paths that the configurations above do not reach: a table codebook (look-up decode kernels up
    to 5 tokens, plain f32 kernels beyond, table GEMM), a densely stored shared expert (extra launches behind the
    routed experts' kernels; the general GEMM on the side stream), a GGUF layer in mixed block types."""
    import torch
    from gfx1151_engine_amd import synth as S
    rng = np.random.default_rng(50 + T)
    d, mid, E, k = 1024, 256, 16, 4
    if variant == "table":
        hl = HostLayer(rng, d, mid, E, k, codebook=S.UNIVERSAL_CODEBOOK, scale_std=0.05)
    elif variant == "dense":
        hl = HostLayer(rng, d, mid, E, k, shared_dense="q8g32")
    else:
        hl = HostLayer(rng, d, mid, E, k, fmt="q4k", gg_types=(13, 8, 12))
    m, dev = hl.to_gpu(max_tokens=64)
    xs = [torch.from_numpy(rng.standard_normal((T, d), dtype=np.float32)).cuda() for _ in range(2)]
    x = torch.empty((T, d), dtype=torch.float32, device="cuda")
    y = torch.empty((T, d), dtype=torch.float32, device="cuda")
    eager = []
    for xi in xs:
        x.copy_(xi)
        m.forward(0, x, y)
        eager.append(y.clone())
    torch.cuda.synchronize()
    want, _, _ = oracle.moe_layer(hl.oracle_layer(), xs[0].cpu().numpy())
    assert np.abs(eager[0].cpu().numpy() - want).max() <= 2e-3 * np.abs(want).max()
    g = torch.cuda.CUDAGraph()
    x.copy_(xs[0])
    with torch.cuda.graph(g):
        m.forward(0, x, y)
    for rep in range(2):
        for i, xi in enumerate(xs):
            x.copy_(xi)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager[i]), (rep, i)
            y.zero_()
            m.forward(0, xs[1 - i], y)
            torch.cuda.synchronize()
            assert torch.equal(y, eager[1 - i])
    m.close()
