"""The benchmark configurations at their full shape (d=3072, mid=768, 512 experts, top-10, shared expert):
the 48-layer stack resident in HBM at one token, the prefill chunks at their full token counts, and the
speculative-verify batch of 20 tokens.  Weights are generated in HBM; the oracle sees the same bytes read
back and evaluates a sample, the rest is covered by properties that do not depend on the size."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu
TOL_LAYER = 2e-3   # max |y - y_ref| / max |y_ref|: f16 MFMA operands, f32 accumulation
TOL_DECODE = 2e-4  # integer-dot decode kernels on q4cp (activations as 16-bit digit planes)
D, MID, E, K = 3072, 768, 512, 10


def _max_abs_rel(y, ref):
    return float(np.abs(y.astype(np.float64) - ref.astype(np.float64)).max() / np.abs(ref).max())


def test_resident_stack_of_48_layers_one_token(oracle):
    """48 x 512 experts (97.8 GB) resident, one token through every layer, each layer with its own weights, routing
    and input.  Router ids of every layer bit-exact with the CPU path; the output of four layers (first, two inner,
    last) within the decode tolerance of the oracle; the whole stack captured as ONE HIP graph replays to the
    eager results bit for bit, with eager calls in between."""
    import torch
    from gfx1151_engine_amd import capi, workloads as W
    NL = 48
    layers = [W.DeviceLayer(3000 + l, D, MID, E, K, "q4cp") for l in range(NL)]
    m = capi.Moe(D, MID, E, K, layers=NL, max_tokens=1)
    for l, L in enumerate(layers):
        L.register(m, l)
    g = torch.Generator(device="cuda")
    g.manual_seed(48)
    x = torch.randn((NL, 1, D), device="cuda", generator=g)
    y = torch.empty((NL, 1, D), dtype=torch.float32, device="cuda")
    ids_all = []
    for l in range(NL):
        m.forward(l, x[l], y[l])
        ids, ws = m.last_routing(1)
        ids_all.append((ids.cpu().numpy()[0, :K].copy(), ws.cpu().numpy()[0, :K].copy()))
    torch.cuda.synchronize()
    eager = y.clone()
    assert torch.isfinite(eager).all()
    xh = x.cpu().numpy()
    seen = set()
    for l in range(NL):  # routing of every layer: the router matrix alone decides it
        lo, io, wo = oracle.router(oracle.Mat(oracle.F32, layers[l].router.cpu().numpy(), E, D), xh[l], K)
        assert (ids_all[l][0] == io[0, :K]).all(), f"layer {l}: router ids"
        assert np.abs(ids_all[l][1] - wo[0, :K]).max() <= 1e-6, f"layer {l}: router weights"
        seen.add(tuple(io[0, :K]))
    assert len(seen) > NL // 2, "the layers route independently"
    for l in (0, 17, 30, NL - 1):  # whole layer against the oracle (2 GB of weights to the host per layer)
        yo, io, wo = oracle.moe_layer(oracle.layer_from_device(layers[l]), xh[l])
        err = _max_abs_rel(eager[l].cpu().numpy(), yo)
        assert err <= TOL_DECODE, (l, err)
    # the reference replays its decode step as a captured graph (src/gpu/parts/40_model.inc:8011-8016,8699-8713)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for l in range(NL):
            m.forward(l, x[l], y[l])
    for rep in range(3):
        y.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {rep}"
        l = (7 * rep + 3) % NL  # eager work between replays, on the same scratch
        y[l].zero_()
        m.forward(l, x[l], y[l])
        torch.cuda.synchronize()
        assert torch.equal(y[l], eager[l])
    m.close()


# "ggmix": the GGUF type mix of the reference's checkpoints (Q5_K gate/up, Q8_0 down, Q8_0 shared expert);
# "i4r": hgn v2 rotated experts with a q4cp shared expert
GG_MIX = (13, 8, 8)


def _device_layer(W, seed, fmt):
    if fmt == "ggmix":
        return W.DeviceLayer(seed, D, MID, E, K, "q4k", gg_types=GG_MIX)
    return W.DeviceLayer(seed, D, MID, E, K, fmt)


@pytest.mark.parametrize("fmt,T", [("q4cp", 16384), ("q4k", 8192), ("q4cp", 3001), ("ggmix", 8192), ("i4r", 16384)])
def test_prefill_chunk_at_full_token_count(oracle, fmt, T):
    """The prefill configurations themselves (T = 16384 q4cp, T = 8192 Q4_K; 3001 for a ragged batch; the same
    chunks for the Q5_K / Q8_0 mix and for hgn v2 rotated experts), Zipf-skewed routing.  Whole batch: ids distinct and in range, weights descending with sum 1, the skew is there, every output
    finite, and each token's result is independent of its position in the batch (the reversed batch gives the
    reversed output bit for bit).  Oracle on a sample: ids and weights bit-exact, output within 2e-3."""
    import torch
    from gfx1151_engine_amd import capi, workloads as W
    L = _device_layer(W, 5151 + T, fmt)
    g = torch.Generator(device="cuda")
    g.manual_seed(T)
    x = torch.randn((T, D), device="cuda", generator=g).to(torch.bfloat16).to(torch.float32)
    L.bias, _ = W.calibrate_zipf(L.router, x, K)
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=T)
    L.register(m, 0)
    y = m.forward(0, x)
    ids, ws = m.last_routing(T)
    yh, ids, ws = y.cpu().numpy(), ids.cpu().numpy()[:, :K], ws.cpu().numpy()[:, :K]
    assert np.isfinite(yh).all()
    srt = np.sort(ids, axis=1)
    assert (srt[:, 1:] != srt[:, :-1]).all() and ids.min() >= 0 and ids.max() < E
    assert np.abs(ws.sum(1) - 1.0).max() < 1e-6 and (np.diff(ws, axis=1) <= 0).all()
    cnt = np.bincount(ids.reshape(-1), minlength=E)
    assert cnt.max() > 8 * cnt.mean(), "hottest expert ~12x the mean"
    # position independence: other tiles, other tile rows, same numbers
    yr = m.forward(0, x.flip(0).contiguous())
    assert torch.equal(yr.flip(0), y), "a token's output must not depend on where it sits in the batch"
    hot, rare = int(np.argmax(cnt)), int(np.argmin(np.where(cnt > 0, cnt, 1 << 30)))
    rs = np.random.default_rng(T)
    sample = np.unique(np.concatenate([np.where((ids == hot).any(1))[0][:6], np.where((ids == rare).any(1))[0][:4],
                                       np.array([0, 1, T // 2, T - 2, T - 1]), rs.integers(0, T, 9)]))
    xs = x[torch.from_numpy(sample).cuda()].contiguous()
    yo, io, wo = oracle.moe_layer(oracle.layer_from_device(L), xs.cpu().numpy())
    assert (ids[sample] == io[:, :K]).all(), "router ids bit-exact with the CPU path"
    assert np.abs(ws[sample] - wo[:, :K]).max() <= 2.5e-7, "router weights: the last bit or two (candidate router)"
    # the dense fp64 router gives the reference's weights bit for bit, and the same experts
    m.set_option(capi.OPT_ROUTER_CANDIDATES, 0)
    m.forward(0, x)
    ids2, ws2 = m.last_routing(T)
    ids2, ws2 = ids2.cpu().numpy()[:, :K], ws2.cpu().numpy()[:, :K]
    assert (ids2 == ids).all(), "candidate router and dense router pick the same experts for every token"
    assert (ws2[sample].view(np.uint32) == wo[:, :K].view(np.uint32)).all(), "dense router: weights bit-exact"
    assert np.abs(ws2 - ws).max() <= 2.5e-7
    err = _max_abs_rel(yh[sample], yo)
    assert err <= TOL_LAYER, err
    m.close()


@pytest.mark.parametrize("uq", [12, 0])  # (12: the distinct-expert path at this size; the default threshold is 24)
def test_verify_batch_of_20_tokens_at_512_experts(oracle, uq):
    """Speculative-verify batch: 4 requests x (4 drafted + 1) = 20 tokens, about 30 % of them reproducing one token's
    top-10 set.  Ids bit-exact, output within the decode tolerance, on the distinct-expert path and with every
    token reading its own experts (MOE_OPT_UNIQUE_MIN_TOKENS = 0, the default at 20 tokens)."""
    import torch
    from gfx1151_engine_amd import capi, workloads as W
    T = 20
    L = W.DeviceLayer(2020, D, MID, E, K, "q4cp")
    m = capi.Moe(D, MID, E, K, layers=1, max_tokens=T)
    L.register(m, 0)
    m.set_option(capi.OPT_UNIQUE_MIN_TOKENS, uq)
    ol = oracle.layer_from_device(L)
    for seed in (5, 6):
        x = W.verify_batch(L.router, D, T, share=0.3, k=K, seed=seed)
        y = m.forward(0, x).cpu().numpy()
        ids, ws = m.last_routing(T)
        ids, ws = ids.cpu().numpy()[:, :K], ws.cpu().numpy()[:, :K]
        yo, io, wo = oracle.moe_layer(ol, x.cpu().numpy())
        assert (ids == io[:, :K]).all()
        assert np.abs(ws - wo[:, :K]).max() <= 1e-6
        shared_set = sum(set(ids[t]) == set(ids[0]) for t in range(T))
        assert shared_set >= 5, "about 30 % of the tokens share the template's experts"
        assert np.unique(ids).size < T * K - 30
        err = _max_abs_rel(y, yo)
        assert err <= TOL_DECODE, err
    m.close()
