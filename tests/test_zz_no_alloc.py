"""moe_routing_run_static (the permutation on the library's fixed device scratch, for callers that cannot
allocate) against moe_routing_run, through the C ABI: bit-exact on two calls in a row, the second smaller; then the same entry point captured into a HIP graph (after the
eager calls, which did the per-device set-up) and replayed on fresh inputs."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _ids(rng, P, E, k):
    ids = np.zeros((P, 16), np.int32)
    ws = np.zeros((P, 16), np.float32)
    pr = 1.0 / (np.arange(E) + 1.0) ** 1.1
    pr[-3:] = 0
    pr /= pr.sum()
    for t in range(P):
        ids[t, :k] = rng.choice(E, k, replace=False, p=pr)
        ws[t, :k] = rng.random(k)
    return ids, ws


def test_static_scratch_routing_equals_routing_run():
    import torch
    from gfx1151_engine_amd import capi
    L = capi.lib()
    assert torch.cuda.is_available()
    E, k = 512, 10
    rng = np.random.default_rng(77)
    r = capi.Routing(6000 * k, E)
    # larger first, then smaller (the scratch keeps the first call's histograms), then a batch of the one-launch size
    for P in (6000, 700, 20):
        ids, ws = _ids(rng, P, E, k)
        gi, gw = torch.from_numpy(ids).cuda(), torch.from_numpy(ws).cuda()
        want = [a.cpu().numpy() for a in r.run(gi, gw, k)]
        n = P * k
        tokidx = torch.full((n,), -1, dtype=torch.int32, device="cuda")
        pw = torch.zeros((n,), dtype=torch.float32, device="cuda")
        eoff = torch.full((E + 1,), -1, dtype=torch.int32, device="cuda")
        pairids = torch.full((n,), -1, dtype=torch.int32, device="cuda")
        torch.cuda.synchronize()
        free0 = torch.cuda.mem_get_info()[0]
        capi.check(L.moe_routing_run_static(capi.ptr(gi), capi.ptr(gw), capi.ptr(tokidx), capi.ptr(pw), capi.ptr(eoff),
                                            capi.ptr(pairids), P, k, E, 16, capi.stream()), "moe_routing_run_static")
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free0, "the call must not change the device's free memory"
        for name, a, b in zip(("tokidx", "pw", "eoff", "pairids"), (tokidx, pw, eoff, pairids), want):
            assert (a.cpu().numpy().view(np.int32) == b.view(np.int32)).all(), (P, name)
    # the wrapper in capi.py gives the same
    got = capi.routing_run_static(gi, gw, k, E)
    for a, b in zip(got, want):
        assert (a.cpu().numpy().view(np.int32) == b.view(np.int32)).all()
    # beyond the fixed scratch: refused, nothing enqueued
    big = torch.zeros((capi.ROUTING_STATIC_MAX_TOKENS + 1, 16), dtype=torch.int32, device="cuda")
    with pytest.raises(capi.MoeError):
        capi.routing_run_static(big, big.float(), k, E)
    r.close()


def test_static_scratch_routing_replays_from_a_graph():
    """Once a call outside a capture has looked the scratch up, the entry point only launches kernels: a captured
    call replays on new ids with the results of moe_routing_run, with eager work between the replays."""
    import torch
    from gfx1151_engine_amd import capi
    L = capi.lib()
    E, k, P = 512, 10, 700
    rng = np.random.default_rng(78)
    r = capi.Routing(P * k, E)
    n = P * k
    gi = torch.zeros((P, 16), dtype=torch.int32, device="cuda")
    gw = torch.zeros((P, 16), dtype=torch.float32, device="cuda")
    tokidx = torch.full((n,), -1, dtype=torch.int32, device="cuda")
    pw = torch.zeros((n,), dtype=torch.float32, device="cuda")
    eoff = torch.full((E + 1,), -1, dtype=torch.int32, device="cuda")
    pairids = torch.full((n,), -1, dtype=torch.int32, device="cuda")

    def call():
        capi.check(L.moe_routing_run_static(capi.ptr(gi), capi.ptr(gw), capi.ptr(tokidx), capi.ptr(pw), capi.ptr(eoff),
                                            capi.ptr(pairids), P, k, E, 16, capi.stream()), "moe_routing_run_static")

    # the set-up call outside any capture (P = 0 is enough)
    capi.check(L.moe_routing_run_static(capi.ptr(gi), capi.ptr(gw), capi.ptr(tokidx), capi.ptr(pw), capi.ptr(eoff),
                                        capi.ptr(pairids), 0, k, E, 16, capi.stream()), "moe_routing_run_static")
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        call()
    for rep in range(3):
        ids, ws = _ids(rng, P, E, k)
        gi.copy_(torch.from_numpy(ids))
        gw.copy_(torch.from_numpy(ws))
        for t in (tokidx, pw, eoff, pairids):
            t.fill_(-1)
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        want = [a.cpu().numpy() for a in r.run(gi, gw, k)]   # eager work between the replays
        for name, a, b in zip(("tokidx", "pw", "eoff", "pairids"), (tokidx, pw, eoff, pairids), want):
            assert (a.cpu().numpy().view(np.int32) == b.view(np.int32)).all(), (rep, name)
    r.close()
