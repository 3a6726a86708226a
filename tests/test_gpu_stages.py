"""GPU parity, stage by stage, through the C ABI: dequantisation and routing bit-exact with the
oracle; the permutation exact; the small-batch GEMV stages within f32 rounding of the oracle."""
import numpy as np
import pytest

from gfx1151_engine_amd import synth as S
from helpers import bits

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def capi():
    import torch
    from gfx1151_engine_amd import capi as c
    c.lib()
    assert torch.cuda.is_available()
    return c


def gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same_bits(a, b):
    a, b = bits(a), bits(b)
    nan = np.isnan(a.view(np.float32)) & np.isnan(b.view(np.float32))
    return bool(((a == b) | nan).all())


# ---------- dequant: bit-exact ----------
def test_q4cp_dequant_golden_and_oracle(capi, oracle, golden):
    g = golden("q4cp_rows.npz")
    for i in range(int(g["n"])):
        rows, cols = (int(v) for v in g[f"shape{i}"])
        got = capi.q4cp_dequant_rows(gpu(g[f"blob{i}"]), rows, cols, 0, rows).cpu().numpy()
        assert same_bits(got, g[f"bits{i}"].view(np.float32)), f"golden case {i}"
    rng = np.random.default_rng(101)
    rows, cols = 512, 3072
    blob = S.make_q4cp(rng, rows, cols, codebook=rng.standard_normal(16).astype(np.float32), scale_std=0.3)
    got = capi.q4cp_dequant_rows(gpu(blob), rows, cols, 100, 300).cpu().numpy()
    assert same_bits(got, oracle.q4cp_rows(blob, rows, cols, 100, 300))
    # empty request is a no-op
    assert capi.q4cp_dequant_rows(gpu(blob), rows, cols, 0, 0).numel() == 0


def test_q4k_dequant_golden_and_oracle(capi, oracle, golden):
    g = golden("q4k_rows.npz")
    for i in range(int(g["n"])):
        rows, cols = (int(v) for v in g[f"shape{i}"])
        got = capi.q4k_dequant_rows(gpu(g[f"raw{i}"]), rows, cols).cpu().numpy()
        assert same_bits(got, g[f"bits{i}"].view(np.float32)), f"golden case {i}"
    rng = np.random.default_rng(102)
    raw = S.make_q4k(rng, 64, 3072, scale_std=0.5)
    assert same_bits(capi.q4k_dequant_rows(gpu(raw), 64, 3072).cpu().numpy(), oracle.q4k_rows(raw, 64, 3072))


def test_q4k_all_scale_min_codes(capi, oracle):
    """Every (sc, m) in [0,63]^2 x q in [0,15] for one block position: brute force."""
    blocks = []
    for sc in range(64):
        q12 = S.pack_scale_min_k4(np.full((64, 8), sc, np.uint8), np.tile(np.arange(64, dtype=np.uint8)[:, None], (1, 8)))
        blk = np.zeros((64, 144), np.uint8)
        blk[:, 0:2] = np.array([0x2E66], np.uint16).view(np.uint8)  # d = 0.1
        blk[:, 2:4] = np.array([0x3266], np.uint16).view(np.uint8)  # dmin = 0.2
        blk[:, 4:16] = q12
        blk[:, 16:] = (np.arange(128) % 16 * 17).astype(np.uint8)
        blocks.append(blk)
    raw = np.concatenate(blocks).reshape(-1)
    n = 64 * 64
    assert same_bits(capi.q4k_dequant_rows(gpu(raw), n, 256).cpu().numpy(), oracle.q4k_rows(raw, n, 256))


@pytest.mark.parametrize("t,cols", [(13, 768), (8, 96), (7, 96), (8, 3072), (7, 768), (12, 512), (20, 96), (20, 768), (23, 768)])
def test_gg_dequant_other_types(capi, oracle, t, cols):
    """Q5_K / Q8_0 / Q5_1 (and Q4_K through the same entry point): bit-exact with the oracle's rows, which the
    CPU tests pin against the reference's gguf::dequant_row; random bytes in the integer fields, so every code
    value occurs."""
    rng = np.random.default_rng(t * 1000 + cols)
    rows = 37
    raw = S.make_gg(rng, t, rows, cols)
    got = capi.gg_dequant_rows(t, gpu(raw), rows, cols).cpu().numpy()
    assert same_bits(got, oracle.gg_rows(t, raw, rows, cols))
    with pytest.raises(capi.MoeError):
        capi.gg_dequant_rows(t, gpu(raw), 1, 48)  # not a whole number of blocks
    with pytest.raises(capi.MoeError):
        capi.gg_dequant_rows(14, gpu(raw), 1, 256)  # Q6_K: outside the path


# ---------- router: bit-exact ----------
@pytest.mark.parametrize("P,E,d,k,dt,mode", [
    (1, 512, 3072, 10, "f32", 0), (20, 512, 3072, 10, "f32", 0), (20, 512, 3072, 10, "f32", 1),
    (300, 512, 3072, 10, "bf16", 0), (77, 96, 200, 5, "f32", 0), (5, 1000, 512, 15, "bf16", 0)])
def test_router_bit_exact(capi, oracle, P, E, d, k, dt, mode):
    rng = np.random.default_rng(1000 + P + E)
    W = rng.standard_normal((E, d), dtype=np.float32) * 0.02
    x = rng.standard_normal((P, d), dtype=np.float32)
    bias = (rng.standard_normal(E) * 0.5).astype(np.float32) if P == 300 else None
    if dt == "bf16":
        wb = S.f32_to_bf16_bits(W)
        Wm = oracle.Mat(oracle.BF16, wb, E, d)
        Wv = capi.wview(gpu(wb.view(np.int16)), capi.BF16, E, d)
    else:
        Wm = oracle.Mat(oracle.F32, W, E, d)
        Wv = capi.wview(gpu(W), capi.F32, E, d)
    lo, io, wo = oracle.router(Wm, x, k, bias=bias)
    lg = capi.router_logits(Wv, gpu(x), gpu(bias) if bias is not None else None, mode)
    ids, ws = capi.router_topk(lg, k)
    lg, ids, ws = lg.cpu().numpy(), ids.cpu().numpy(), ws.cpu().numpy()
    assert (ids[:, :k] == io[:, :k]).all(), "expert ids / order differ"
    if mode == 1 or P > 32:
        assert same_bits(lg, lo), "sequential-order logits must be bit-identical"
        assert same_bits(ws[:, :k], wo[:, :k])
    else:
        assert np.abs(lg - lo).max() <= 2.4e-7 * np.abs(lo).max() + 1e-12  # at most the last f32 bit
        assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 1e-6


def test_router_topk_ties_and_wide_range(capi, oracle):
    import torch
    E, k = 512, 10
    rows = [np.zeros(E, np.float32)]                      # all equal -> ids 0..9
    r = np.zeros(E, np.float32); r[300] = 40.0; rows.append(r)       # one-hot, rest tie
    r = np.repeat(np.arange(E // 2, dtype=np.float32), 2)[::-1].copy() * 0.01; rows.append(r)  # equal pairs
    r = np.linspace(0, -90, E, dtype=np.float32); rows.append(r)     # range > 13.8: sequential-sum fallback
    r = np.linspace(0, -200, E, dtype=np.float32); rows.append(r)    # underflow to zero probabilities
    lg = np.stack(rows)
    ids, ws = capi.router_topk(gpu(lg), k)
    ids, ws = ids.cpu().numpy(), ws.cpu().numpy()
    for t in range(lg.shape[0]):
        p, io, wo = oracle.softmax_topk(lg[t], k)
        assert (ids[t, :k] == io).all(), t
        assert same_bits(ws[t, :k], wo), t
    assert list(ids[0, :k]) == list(range(10))


# ---------- permutation: exact ----------
@pytest.mark.parametrize("P,E,k", [(1, 512, 10), (20, 512, 10), (32, 512, 10), (33, 512, 10), (32, 20, 16), (255, 512, 10), (257, 40, 6), (5000, 512, 10), (3, 7, 7)])
def test_routing_exact(capi, oracle, P, E, k):
    rng = np.random.default_rng(P * 7 + E)
    ids = np.zeros((P, 16), np.int32)
    ws = np.zeros((P, 16), np.float32)
    # skewed choice so that some experts are empty and some are hot
    pr = 1.0 / (np.arange(E) + 1.0) ** 1.1
    pr[-3:] = 0 if E > 10 else pr[-3:]
    pr /= pr.sum()
    for t in range(P):
        ids[t, :k] = rng.choice(E, k, replace=False, p=pr if E > 10 else None)
        ws[t, :k] = rng.random(k)
    r = capi.Routing(P * k, E)
    tokidx, pw, eoff, pairids = (a.cpu().numpy() for a in r.run(gpu(ids), gpu(ws), k))
    to, po, eo, qo = oracle.route(ids, ws, k, E)
    assert (eoff == eo).all() and (tokidx == to).all() and (pw == po).all() and (pairids == qo).all()
    for cap in (64, 128):
        t, n = capi.tiles(gpu(eo), cap, P * k)
        want = oracle.tiles(eo, cap)
        n = int(n.item())
        assert n == want.shape[0] and (t.cpu().numpy()[:n] == want).all()
    r.close()


def test_routing_capacity_and_empty(capi):
    import torch
    r = capi.Routing(100, 16)
    ids = torch.zeros((20, 16), dtype=torch.int32, device="cuda")
    ws = torch.zeros((20, 16), dtype=torch.float32, device="cuda")
    with pytest.raises(capi.MoeError):
        r.run(ids, ws, 10)  # 200 pairs > capacity
    tokidx, pw, eoff, _ = r.run(ids[:0], ws[:0], 10)
    assert (eoff.cpu().numpy() == 0).all()
    r.close()


# ---------- small-batch GEMV stages ----------
@pytest.mark.parametrize("d,mid,E,k,P,cbkind", [(3072, 768, 16, 10, 3, "zp8"), (640, 160, 8, 4, 5, "random"),
                                                (256, 96, 6, 2, 2, "zp8")])
def test_q4cp_gemv_stages(capi, oracle, d, mid, E, k, P, cbkind):
    rng = np.random.default_rng(d + mid)
    cb = None if cbkind == "zp8" else rng.uniform(-2, 2, 16).astype(np.float32)
    gu = S.make_q4cp(rng, E * 2 * mid, d, codebook=cb, scale_std=0.02)
    dn = S.make_q4cp(rng, E * d, mid, codebook=cb, scale_std=0.02)
    x = rng.standard_normal((P, d), dtype=np.float32)
    ids = np.zeros((P, 16), np.int32)
    ws = np.zeros((P, 16), np.float32)
    for t in range(P):
        ids[t, :k] = rng.choice(E, k, replace=False)
        w = rng.random(k).astype(np.float32)
        ws[t, :k] = w / w.sum()
    guv = capi.wview(gpu(gu), capi.Q4CP, E * 2 * mid, d)
    dnv = capi.wview(gpu(dn), capi.Q4CP, E * d, mid)
    hid = capi.q4cp_gemv_gate_up(guv, gpu(x), gpu(ids), k, mid)
    ey = rng.standard_normal((P, d), dtype=np.float32)
    sg = rng.standard_normal(P).astype(np.float32)
    y = capi.q4cp_gemv_down_topk(dnv, hid, gpu(ids), gpu(ws), k, d).cpu().numpy()
    y2 = capi.q4cp_gemv_down_topk(dnv, hid, gpu(ids), gpu(ws), k, d, gpu(ey), gpu(sg)).cpu().numpy()
    hid = hid.cpu().numpy().reshape(P, k, mid)
    # fp64 evaluation from the oracle's dequantised rows
    GU = oracle.q4cp_rows(gu, E * 2 * mid, d, 0, E * 2 * mid).astype(np.float64)
    DN = oracle.q4cp_rows(dn, E * d, mid, 0, E * d).astype(np.float64)
    for t in range(P):
        acc = np.zeros(d)
        for s in range(k):
            e = ids[t, s]
            g = (GU[e * 2 * mid:e * 2 * mid + mid] @ x[t]).astype(np.float32)
            u = (GU[e * 2 * mid + mid:(e + 1) * 2 * mid] @ x[t]).astype(np.float32)
            h = (g / (1 + np.exp(-g.astype(np.float64)))).astype(np.float32) * u
            assert np.abs(hid[t, s] - h).max() <= 1e-4 * np.abs(h).max(), (t, s)  # reference: rel 1e-4
            acc += float(ws[t, s]) * (DN[e * d:(e + 1) * d] @ hid[t, s].astype(np.float64))
        assert np.abs(y[t] - acc).max() <= 1e-4 * np.abs(acc).max()
        want2 = acc + ey[t] / (1 + np.exp(-float(sg[t])))
        assert np.abs(y2[t] - want2).max() <= 1e-4 * np.abs(want2).max()


def test_gemv_row_invariance(capi):
    """The result for a token must not depend on the batch it is in (reference: ktest 'ri_' cases)."""
    rng = np.random.default_rng(9)
    d, mid, E, k, P = 1024, 256, 12, 4, 7
    gu = gpu(S.make_q4cp(rng, E * 2 * mid, d))
    dn = gpu(S.make_q4cp(rng, E * d, mid))
    x = gpu(rng.standard_normal((P, d), dtype=np.float32))
    ids = np.zeros((P, 16), np.int32)
    ws = np.zeros((P, 16), np.float32)
    for t in range(P):
        ids[t, :k] = rng.choice(E, k, replace=False)
        ws[t, :k] = 1.0 / k
    ids, ws = gpu(ids), gpu(ws)
    guv, dnv = capi.wview(gu, capi.Q4CP, E * 2 * mid, d), capi.wview(dn, capi.Q4CP, E * d, mid)
    hid = capi.q4cp_gemv_gate_up(guv, x, ids, k, mid)
    y = capi.q4cp_gemv_down_topk(dnv, hid, ids, ws, k, d)
    for t in (0, 3, 6):
        h1 = capi.q4cp_gemv_gate_up(guv, x[t:t + 1].contiguous(), ids[t:t + 1].contiguous(), k, mid)
        y1 = capi.q4cp_gemv_down_topk(dnv, h1, ids[t:t + 1].contiguous(), ws[t:t + 1].contiguous(), k, d)
        assert (h1.view(-1) == hid.view(P, -1)[t]).all() and (y1[0] == y[t]).all()


# ---------- batch router through candidate selection ----------
def _route_both(capi, hl, x, k):
    """(ids, ws) of the batch path with the candidate router and with the dense fp64 router."""
    import torch
    T = x.shape[0]
    m, dev = hl.to_gpu(max_tokens=T)
    out = []
    for opt in (1, 0):
        m.set_option(capi.OPT_ROUTER_CANDIDATES, opt)
        m.forward(0, gpu(x))
        ids, ws = m.last_routing(T)
        out.append((ids.cpu().numpy()[:, :k].copy(), ws.cpu().numpy()[:, :k].copy()))
    m.close()
    return out


@pytest.mark.parametrize("E,k,d,T,dt", [(512, 10, 3072, 700, "f32"), (512, 10, 1024, 300, "bf16"), (64, 6, 256, 130, "f32"),
                                        (40, 15, 512, 77, "f32"), (500, 8, 640, 100, "bf16"), (600, 8, 384, 90, "f32"),
                                        (96, 4, 320, 70, "f32"), (1000, 10, 256, 65, "bf16")])
def test_candidate_router_ids_exact(capi, oracle, E, k, d, T, dt):
    """Approximate logits + rigorous bound + exact recomputation of the candidates: ids and their order are the
    oracle's for every token, weights within the last bit or two, with and without a Zipf bias.  (d = 320 is a shape
    the batch path refuses: the library walks the batch through the in-place path 32 rows at a time, and the router
    output it keeps must still cover every row.)"""
    from helpers import HostLayer
    rng = np.random.default_rng(E + T)
    for skew in (False, True):
        bias = S.zipf_bias(rng, E, 1.1, 1.0) if skew else None
        hl = HostLayer(rng, d, 256, E, k, router_dtype=dt, bias=bias, shared=(T % 2 == 0))
        x = rng.standard_normal((T, d), dtype=np.float32) * (0.3 if skew else 3.0)
        lo, io, wo = oracle.router(hl.oracle_layer().router, x, k, bias=bias)
        (ic, wc), (i0, w0) = _route_both(capi, hl, x, k)
        assert (i0 == io[:, :k]).all() and (w0.view(np.uint32) == wo[:, :k].view(np.uint32)).all(), "dense router"
        assert (ic == io[:, :k]).all(), "candidate router: ids / order differ from the oracle"
        assert np.abs(wc - wo[:, :k]).max() <= 2.5e-7


def test_candidate_router_hard_rows(capi, oracle):
    """Rows that the candidate pass must hand to the exact redo: duplicated and nearly equal router rows (probability
    ties at and around the rank k boundary), all-zero tokens (every logit equal), a logit range of hundreds (f32
    probabilities underflow and tie by index), activations beyond the f16 range, and a batch in which most tokens are
    such (the dense kernel takes over).  Ids must be the oracle's everywhere."""
    from helpers import HostLayer
    rng = np.random.default_rng(404)
    E, k, d, T = 128, 10, 512, 200
    hl = HostLayer(rng, d, 256, E, k, shared=False)
    hl.router[7] = hl.router[3]
    hl.router[90] = hl.router[3]
    hl.router[16] = hl.router[5] * np.float32(1 + 2 ** -22)
    hl.router[33] = hl.router[5]
    x = rng.standard_normal((T, d), dtype=np.float32)
    x[10] = 0.0
    x[11] = 0.0
    x[12] *= 300.0                      # logits spread over hundreds
    x[13] = x[12] * 40.0
    x[14, 5] = 1e5                      # beyond f16
    x[15] *= 1e-6                       # f16 subnormals
    for sel in (slice(None), np.r_[0:40, 10, 11, 10, 11, 10, 11, 12, 13]):
        xs = np.ascontiguousarray(x[sel])
        lo, io, wo = oracle.router(hl.oracle_layer().router, xs, k)
        (ic, wc), (i0, w0) = _route_both(capi, hl, xs, k)
        assert (i0 == io[:, :k]).all()
        assert (ic == io[:, :k]).all(), np.where((ic != io[:, :k]).any(1))
        assert np.abs(wc - wo[:, :k]).max() <= 2.5e-7
    # most tokens tie: every token is listed and the dense kernel runs
    xz = np.zeros((64, d), np.float32)
    xz[::7] = x[:10]
    lo, io, wo = oracle.router(hl.oracle_layer().router, xz, k)
    (ic, wc), _ = _route_both(capi, hl, xz, k)
    assert (ic == io[:, :k]).all() and (wc.view(np.uint32) == wo[:, :k].view(np.uint32)).all()
