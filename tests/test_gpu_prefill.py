"""GPU parity of the batch (prefill) path: MFMA grouped GEMM stages against fp64 evaluations of the
oracle's dequantised weights, and the whole layer against the oracle within max-abs-rel 2e-3."""
import numpy as np
import pytest

from gfx1151_engine_amd import synth as S
from helpers import HostLayer, max_abs_rel

pytestmark = pytest.mark.gpu
TOL_LAYER = 2e-3  # north-star tolerance: f16 MFMA operands, f32 accumulation, vs the fp64/f32 CPU path


def gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def capi():
    from gfx1151_engine_amd import capi as c
    c.lib()
    return c


def make_routing(rng, P, E, k, counts=None):
    ids = np.zeros((P, 16), np.int32)
    ws = np.zeros((P, 16), np.float32)
    for t in range(P):
        ids[t, :k] = rng.choice(E, k, replace=False)
        w = rng.random(k).astype(np.float32) + 0.1
        ws[t, :k] = w / w.sum()
    return ids, ws


@pytest.mark.parametrize("d,mid,E,k,P,cb", [(256, 256, 6, 2, 300, "zp8"), (640, 384, 4, 2, 260, "zp8"), (3072, 768, 8, 4, 200, "zp8"),
                                            (512, 256, 5, 3, 150, "random")])
def test_grouped_gemm_stages(capi, oracle, d, mid, E, k, P, cb):
    """up -> hid16, down -> pairs, reduce -> y, each against fp64 from the oracle's weights.
    Expert 0 is left empty and one expert gets a 1-pair tile and a 129-pair run (tile edge cases,
    reference: tools/ktest.cu:2588-2592 uses counts {0,1,63,64,65,2})."""
    import torch
    rng = np.random.default_rng(d + P)
    codebook = None if cb == "zp8" else rng.uniform(-2, 2, 16).astype(np.float32)
    gu = S.make_q4cp(rng, E * 2 * mid, d, codebook=codebook, scale_std=0.02)
    dn = S.make_q4cp(rng, E * d, mid, codebook=codebook, scale_std=0.02)
    x = rng.standard_normal((P, d), dtype=np.float32)
    ids, ws = make_routing(rng, P, E - 1, k)
    ids[:, :k] += 1  # expert 0 empty
    x16 = capi.f32_to_f16(gpu(x))
    assert (capi.from_layout1(x16).cpu().numpy() == x.astype(np.float16)).all()
    assert (capi.f32_to_f16(gpu(x), layout=0).cpu().numpy() == x.astype(np.float16)).all()
    r = capi.Routing(P * k, E)
    tokidx, pw, eoff, pairids = r.run(gpu(ids), gpu(ws), k)
    tiles_t, ntiles = capi.tiles(eoff, 128, P * k)
    pgu = capi.lut_q4cp_view(gpu(gu), E * 2 * mid, d, 2 * mid, mid)
    pdn = capi.lut_q4cp_view(gpu(dn), E * d, mid, d, 0)
    hid = capi.lut_up(pgu, x16, tokidx, tiles_t, ntiles, mid, P * k)
    pairs = capi.lut_down(pdn, hid, tiles_t, ntiles, d, f16=False)
    pairs16 = capi.lut_down(pdn, hid, tiles_t, ntiles, d, f16=True)
    y = capi.reduce_pw_sg(pairs, pairids, pw, P, k)
    hid, pairs, pairs16, y = capi.from_layout1(hid).cpu().numpy(), pairs.cpu().numpy(), pairs16.cpu().numpy(), y.cpu().numpy()
    assert not np.isnan(hid).any() and not np.isnan(pairs).any(), "every pair row must be written"
    tokidx, pw, eoff = tokidx.cpu().numpy(), pw.cpu().numpy(), eoff.cpu().numpy()
    GU = oracle.q4cp_rows(gu, E * 2 * mid, d, 0, E * 2 * mid).astype(np.float64)
    DN = oracle.q4cp_rows(dn, E * d, mid, 0, E * d).astype(np.float64)
    x64 = x.astype(np.float16).astype(np.float64)
    yref = np.zeros((P, d))
    for e in range(E):
        sl = slice(eoff[e], eoff[e + 1])
        if sl.start == sl.stop:
            continue
        xe = x64[tokidx[sl]]
        g = xe @ GU[e * 2 * mid:e * 2 * mid + mid].T
        u = xe @ GU[e * 2 * mid + mid:(e + 1) * 2 * mid].T
        h = g / (1 + np.exp(-g)) * u
        assert np.abs(hid[sl] - h).max() <= 3e-3 * np.abs(h).max(), e
        pr = hid[sl].astype(np.float64) @ DN[e * d:(e + 1) * d].T
        assert np.abs(pairs[sl] - pr).max() <= 2e-3 * np.abs(pr).max(), e
        assert np.abs(pairs16[sl] - pr).max() <= 3e-3 * np.abs(pr).max(), e
        np.add.at(yref, tokidx[sl], pw[sl, None].astype(np.float64) * pairs[sl].astype(np.float64))
    assert np.abs(y - yref).max() <= 1e-5 * np.abs(yref).max()
    r.close()


@pytest.mark.parametrize("d,mid,E,k,P", [(256, 256, 6, 2, 300), (768, 512, 4, 2, 260), (3072, 768, 6, 3, 200)])
def test_grouped_gemm_stages_q4k(capi, oracle, d, mid, E, k, P):
    """moe_gg_up / moe_gg_down on raw Q4_K blocks, against fp64 from the oracle's dequantised weights
    (f16 weights and activations: per-element error ~2^-11, so 3e-3 of the row maximum is the bound)."""
    rng = np.random.default_rng(d + P + 1)
    gate = S.make_q4k(rng, E * mid, d, scale_std=0.0005)
    up = S.make_q4k(rng, E * mid, d, scale_std=0.0005)
    dn = S.make_q4k(rng, E * d, mid, scale_std=0.0005)
    x = rng.standard_normal((P, d), dtype=np.float32)
    ids, ws = make_routing(rng, P, E - 1, k)
    ids[:, :k] += 1  # expert 0 empty
    x16 = capi.f32_to_f16(gpu(x), layout=2)
    assert (capi.from_layout2(x16).cpu().numpy() == x.astype(np.float16)).all()
    r = capi.Routing(P * k, E)
    tokidx, pw, eoff, pairids = r.run(gpu(ids), gpu(ws), k)
    tiles_t, ntiles = capi.tiles(eoff, 128, P * k)
    hid = capi.gg_up(gpu(gate), gpu(up), x16, tokidx, tiles_t, ntiles, mid, P * k)
    pairs = capi.gg_down(gpu(dn), hid, tiles_t, ntiles, d, f16=False)
    pairs16 = capi.gg_down(gpu(dn), hid, tiles_t, ntiles, d, f16=True)
    hid, pairs, pairs16 = capi.from_layout2(hid).cpu().numpy(), pairs.cpu().numpy(), pairs16.cpu().numpy()
    assert not np.isnan(hid).any() and not np.isnan(pairs).any(), "every pair row must be written"
    tokidx, eoff = tokidx.cpu().numpy(), eoff.cpu().numpy()
    G = oracle.q4k_rows(gate, E * mid, d).astype(np.float64)
    U = oracle.q4k_rows(up, E * mid, d).astype(np.float64)
    DN = oracle.q4k_rows(dn, E * d, mid).astype(np.float64)
    x64 = x.astype(np.float16).astype(np.float64)
    for e in range(E):
        sl = slice(eoff[e], eoff[e + 1])
        if sl.start == sl.stop:
            continue
        xe = x64[tokidx[sl]]
        g = xe @ G[e * mid:(e + 1) * mid].T
        u = xe @ U[e * mid:(e + 1) * mid].T
        h = g / (1 + np.exp(-g)) * u
        assert np.abs(hid[sl] - h).max() <= 3e-3 * np.abs(h).max(), e
        pr = hid[sl].astype(np.float64) @ DN[e * d:(e + 1) * d].T
        assert np.abs(pairs[sl] - pr).max() <= 3e-3 * np.abs(pr).max(), e
        assert np.abs(pairs16[sl] - pr).max() <= 4e-3 * np.abs(pr).max(), e
    r.close()


def check_fused_combine(m, x, y_ordered, yo):
    """MOE_OPT_FUSED_COMBINE: the down GEMM adds its weighted rows into y (f32 atomics).  Same layer bar; against
    the ordered two-step result only the f16 rounding of the pair rows and the order of the additions differ.
    Run twice: y is zeroed inside every call, so what an earlier call left there must not matter."""
    from gfx1151_engine_amd import capi
    m.set_option(capi.OPT_FUSED_COMBINE, 1)
    for _ in range(2):
        yf = m.forward(0, gpu(x)).cpu().numpy()
        assert max_abs_rel(yf, yo) <= TOL_LAYER, max_abs_rel(yf, yo)
        assert max_abs_rel(yf, y_ordered) <= 1e-3, max_abs_rel(yf, y_ordered)
    m.set_option(capi.OPT_FUSED_COMBINE, 0)
    assert (m.forward(0, gpu(x)).cpu().numpy() == y_ordered).all(), "the ordered form is deterministic"


@pytest.mark.parametrize("d,mid,E,k,T", [(512, 256, 16, 4, 333), (3072, 768, 32, 10, 300)])
def test_batch_layer_vs_oracle_q4k(oracle, d, mid, E, k, T):
    """GGUF Q4_K experts + Q4_K shared expert through the MFMA path."""
    rng = np.random.default_rng(d * 5 + T)
    hl = HostLayer(rng, d, mid, E, k, fmt="q4k")
    x = S.bf16_round(rng.standard_normal((T, d), dtype=np.float32))
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    y = m.forward(0, gpu(x))
    ids, ws = m.last_routing(T)
    y, ids = y.cpu().numpy(), ids.cpu().numpy()
    assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    err = max_abs_rel(y, yo)
    assert err <= TOL_LAYER, err
    check_fused_combine(m, x, y, yo)
    m.close()


@pytest.mark.parametrize("d,mid,E,k,T,skew", [(512, 256, 16, 4, 333, False), (3072, 768, 64, 10, 700, True),
                                              (1024, 256, 8, 3, 33, False)])
def test_batch_layer_vs_oracle(oracle, d, mid, E, k, T, skew):
    rng = np.random.default_rng(d * 3 + T)
    bias = S.zipf_bias(rng, E, 1.1, 1.0) if skew else None
    hl = HostLayer(rng, d, mid, E, k, bias=bias)
    x = S.bf16_round(rng.standard_normal((T, d), dtype=np.float32))
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    y = m.forward(0, gpu(x))
    ids, ws = m.last_routing(T)
    y, ids, ws = y.cpu().numpy(), ids.cpu().numpy(), ws.cpu().numpy()
    assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 2.5e-7, "router weights within the last bit or two"
    from gfx1151_engine_amd import capi
    m.set_option(capi.OPT_ROUTER_CANDIDATES, 0)   # dense fp64 router: the reference's weights bit for bit
    y0 = m.forward(0, gpu(x)).cpu().numpy()
    ids0, ws0 = m.last_routing(T)
    assert (ids0.cpu().numpy()[:, :k] == io[:, :k]).all()
    assert (ws0.cpu().numpy()[:, :k].view(np.uint32) == wo[:, :k].view(np.uint32)).all(), "sequential-order router weights are bit-exact"
    assert max_abs_rel(y0, yo) <= TOL_LAYER
    m.set_option(capi.OPT_ROUTER_CANDIDATES, 1)
    err = max_abs_rel(y, yo)
    assert err <= TOL_LAYER, err
    check_fused_combine(m, x, y, yo)
    m.close()


@pytest.mark.parametrize("cb,sstd", [("universal", 0.002), ("zp8", 0.0003), ("universal", 0.0005)])
def test_batch_layer_with_very_small_weights(oracle, cb, sstd):
    """Weights several to thirty times smaller than the benchmark's: the down-projection pair rows (about 3e-6 and
    below at unit activations) would sit in f16's subnormal range; the range guard scales such rows up by a power of
    two on their way through f16 and the combine takes it out again."""
    rng = np.random.default_rng(1039)
    d, mid, E, k, T = 256, 384, 32, 4, 108
    hl = HostLayer(rng, d, mid, E, k, codebook=S.UNIVERSAL_CODEBOOK if cb == "universal" else None, scale_std=sstd,
                   shared=(cb == "zp8"), bias=S.zipf_bias(rng, E, 1.1, 1.0))
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, ws = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    err = max_abs_rel(y, yo)
    assert err <= TOL_LAYER, err
    m.close()


@pytest.mark.parametrize("fmt,kw,d,mid,want", [
    ("q4cp", {}, 512, 256, "batch"), ("q4cp", {"codebook": "universal"}, 512, 256, "batch"),
    ("q4cp", {"shared": False}, 256, 384, "batch"), ("q4k", {}, 512, 256, "batch"),
    ("q4k", {"gg_types": (13, 8, 8)}, 512, 256, "batch"), ("q4k", {"gg_types": (23, 20, 12)}, 512, 256, "batch"),
    ("i4r", {}, 512, 256, "batch"), ("i4r", {"shared": False}, 256, 512, "batch"), ("i4r", {"shared_dense": "bf16"}, 512, 256, "batch"),
    ("q4cp", {"shared_dense": "q8g64"}, 512, 256, "batch"),
    ("q4cp", {}, 320, 256, "walked"), ("i4r", {}, 384, 384, "walked")])
def test_which_shapes_take_the_grouped_gemm(oracle, fmt, kw, d, mid, want):
    """moe_last_path: batches over 32 tokens of every supported format run on the grouped GEMM (a launch plan that
    declines silently would send them through the in-place kernels 32 rows at a time -- right results, several times
    the time); shapes outside the GEMM's tiling are walked; at most 32 tokens take the in-place kernels."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(77 + d + mid)
    kw = dict(kw)
    if kw.get("codebook") == "universal":
        kw["codebook"] = S.UNIVERSAL_CODEBOOK
    E, k, T = 8, 2, 70
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt, **kw)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    assert m.last_path() == capi.PATH_NONE
    y = m.forward(0, gpu(x)).cpu().numpy()
    assert m.last_path() == (capi.PATH_BATCH if want == "batch" else capi.PATH_WALKED)
    assert max_abs_rel(y, yo) <= TOL_LAYER, max_abs_rel(y, yo)
    m.forward(0, gpu(x[:7]))
    assert m.last_path() == capi.PATH_SMALL
    m.close()


@pytest.mark.parametrize("sstd,xs,shared", [(0.0005, 0.3, True), (0.0005, 0.3, False), (0.3, 3.0, True), (0.002, 1.0, False)])
def test_batch_layer_of_rotated_experts_with_weights_far_off_the_usual_scale(oracle, sstd, xs, shared):
    """hgn v2 rotated experts twenty times smaller / thirty times larger than usual: the rows between the two
    projections (rotated hid, pair rows) would leave f16's normal range on either side; the range guard applies to
    this path as well (a power of two per token in the slot-wise middle, divided out in the combine)."""
    rng = np.random.default_rng(5032 + int(sstd * 1e4))
    d, mid, E, k, T = 256, 512, 32, 2, 172
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r", scale_std=sstd, shared=shared, bias=S.zipf_bias(rng, E, 1.1, 1.0))
    x = rng.standard_normal((T, d), dtype=np.float32) * xs
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, ws = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    assert np.isfinite(y).all()
    err = max_abs_rel(y, yo)
    assert err <= TOL_LAYER, err
    m.close()


@pytest.mark.parametrize("kind", ["affine", "table", "mixed"])
@pytest.mark.parametrize("T", [70, 20])
def test_shared_expert_with_a_codebook_per_tensor(oracle, kind, T):
    """gate_proj, up_proj and down_proj of the shared expert are separately quantised tensors: each carries its own
    codebook (the reference's converter trains one per dense tensor; only routed experts share one).  Batch path
    (grouped GEMM: gate and up rows in one launch) and small path against the oracle."""
    rng = np.random.default_rng(len(kind) * 100 + T)
    n = np.arange(16, dtype=np.float32)
    if kind == "affine":     # three different uniform grids
        cbs = [n - 8, 0.5 * n - 3.0, -0.25 * n + 1.0]
    elif kind == "table":    # three different non-uniform tables
        cbs = [np.sort(rng.uniform(-2, 2, 16)).astype(np.float32) for _ in range(3)]
    else:                    # gate uniform, up a table, down another grid
        cbs = [n - 8, np.sort(rng.standard_normal(16)).astype(np.float32) * 3, 2 * n - 15]
    d, mid, E, k = 512, 256, 8, 3
    hl = HostLayer(rng, d, mid, E, k, shared_codebooks=[c.astype(np.float32) for c in cbs])
    x = S.bf16_round(rng.standard_normal((T, d), dtype=np.float32))
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    y = m.forward(0, gpu(x))
    ids, _ = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    err = max_abs_rel(y.cpu().numpy(), yo)
    assert err <= TOL_LAYER, err
    m.close()


def test_batch_equals_small_path_statistically(oracle):
    """Same layer through the MFMA path (T=40) and the f32 in-place path (two calls of 20)."""
    rng = np.random.default_rng(5)
    hl = HostLayer(rng, 1024, 256, 12, 4)
    x = rng.standard_normal((40, 1024), dtype=np.float32)
    m, dev = hl.to_gpu(max_tokens=64)
    xb = gpu(x)
    yb = m.forward(0, xb).cpu().numpy()
    ys = np.concatenate([m.forward(0, xb[:20].contiguous()).cpu().numpy(), m.forward(0, xb[20:].contiguous()).cpu().numpy()])
    assert max_abs_rel(yb, ys) <= TOL_LAYER
    m.close()


@pytest.mark.parametrize("fmt", ["q4cp", "q4k"])
def test_forward_hc_writeback(oracle, fmt):
    """moe_forward_hc (the reference's moe_b with try_hcw): the combine adds into the bf16 HC state instead of
    writing f32.  Against the oracle's write-back applied to moe_forward's own output: identical where the gate
    logit is 0 (inj = 1 exactly); elsewhere device and host expf may differ in the last bit of inj, which can move
    a result across a bf16 rounding boundary: at most one bf16 step at the operands' size, in well under 1 % of the
    elements.  Batches
    of at most 32 tokens are refused, as the reference's call returns false there."""
    import torch
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(77)
    d, mid, E, k, T = 512, 256, 12, 4, 150
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt)
    x = S.bf16_round(rng.standard_normal((T, d), dtype=np.float32))
    m, dev = hl.to_gpu(max_tokens=T)
    y = m.forward(0, gpu(x)).cpu().numpy()
    w4 = rng.standard_normal((T, 4)).astype(np.float32) * 2
    w4[:, 0] = 0.0
    R0 = (rng.standard_normal((T, 4, d)).astype(np.float32).view(np.uint32) >> 16).astype(np.uint16)
    want = oracle.hc_writeback(y, w4, R0)
    R = torch.from_numpy(R0.view(np.int16).copy()).cuda()
    m.forward_hc(0, gpu(x), gpu(w4), R)
    got = R.cpu().numpy().view(np.uint16)
    assert (got[:, 0] == want[:, 0]).all()
    gv, wv = ((a.astype(np.uint32) << 16).view(np.float32) for a in (got, want))
    r0 = (R0.astype(np.uint32) << 16).view(np.float32)
    step = 2.0 ** -7 * (np.abs(r0) + 2 * np.abs(y)[:, None, :])  # a bf16 step at the operands' size (sums may cancel)
    assert (np.abs(gv - wv) <= step).all() and (got != want).mean() < 0.01, (got != want).mean()
    with pytest.raises(capi.MoeError):
        m.forward_hc(0, gpu(x[:8]), gpu(w4[:8]), R)
    # stage level: the same kernel behind moe_reduce_pw_sg_hc, no shared expert, f32 pairs
    P2, K2 = 40, 3
    pairs = rng.standard_normal((P2 * K2, d)).astype(np.float32)
    pairids = rng.permutation(P2 * K2).astype(np.int32).reshape(P2, K2)
    pw = rng.random(P2 * K2).astype(np.float32)
    y2 = capi.reduce_pw_sg(gpu(pairs), gpu(pairids), gpu(pw), P2, K2).cpu().numpy()
    R2 = torch.from_numpy(R0[:P2].view(np.int16).copy()).cuda()
    z4 = np.zeros((P2, 4), np.float32)
    capi.reduce_pw_sg_hc(gpu(pairs), gpu(pairids), gpu(pw), P2, K2, gpu(z4), R2)
    assert (R2.cpu().numpy().view(np.uint16) == oracle.hc_writeback(y2, z4, R0[:P2])).all()
    m.close()


@pytest.mark.parametrize("shared", ["same", "per_tensor", "affine", "bf16", "none"])
@pytest.mark.parametrize("d,mid,E,k,T", [(512, 256, 8, 3, 70), (768, 512, 6, 2, 300), (3072, 768, 12, 4, 161)])
def test_batch_layer_with_a_table_codebook(oracle, shared, d, mid, E, k, T):
    """Routed experts with a codebook that is not a*n + b (what the reference's converter writes by default: its
    universal expert codebook): the grouped GEMMs of the layer run in natural K order through pair tables.  The shared
    expert with the same table, a table per tensor, uniform grids, dense bf16 rows, or absent; the shared expert aside
    or in the routed launches, the ordered and the fused combine.  ids bit-exact, output within the batch bar."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(d + T + len(shared))
    n = np.arange(16, dtype=np.float32)
    cb = np.sort(rng.uniform(-2, 2, 16)).astype(np.float32)
    kw = {}
    if shared == "per_tensor":
        kw["shared_codebooks"] = [np.sort(rng.uniform(-2, 2, 16)).astype(np.float32) for _ in range(3)]
    elif shared == "affine":
        kw["shared_codebooks"] = [n - 8, 0.5 * n - 3.0, -0.25 * n + 1.0]
    elif shared == "bf16":
        kw["shared_dense"] = "bf16"
    elif shared == "none":
        kw["shared"] = False
    hl = HostLayer(rng, d, mid, E, k, codebook=cb, **kw)
    x = S.bf16_round(rng.standard_normal((T, d), dtype=np.float32))
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    assert m.x16_layout(0) == 0, "table codebooks: activations in natural order"
    for aside, fused in ((1, 0), (0, 0), (0, 1)):
        m.set_option(capi.OPT_SHARED_ASIDE, aside)
        m.set_option(capi.OPT_FUSED_COMBINE, fused)
        y = m.forward(0, gpu(x))
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
        err = max_abs_rel(y.cpu().numpy(), yo)
        assert err <= TOL_LAYER, (aside, fused, err)
    m.set_option(capi.OPT_SHARED_ASIDE, 1)
    m.set_option(capi.OPT_FUSED_COMBINE, 0)
    y0 = m.forward(0, gpu(x)).cpu().numpy()
    y1 = m.forward_x16(0, gpu(x), capi.f32_to_f16(gpu(x), layout=0)).cpu().numpy()
    assert (y1 == y0).all(), "the caller's natural-order f16 copy gives the same bits"
    m.close()


@pytest.mark.parametrize("fmt", ["q4cp", "q4k"])
def test_forward_with_the_callers_f16_copy(oracle, fmt):
    """moe_forward_x16: the caller hands over the f16 copy of the batch in the grouped GEMM's order (its own epilogue
    wrote it), the library skips its conversion pass.  Same bits as moe_forward; small batches are refused."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(61)
    d, mid, E, k, T = 512, 256, 12, 4, 130
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt)
    x = rng.standard_normal((T, d), dtype=np.float32)
    m, dev = hl.to_gpu(max_tokens=T)
    xg = gpu(x)
    layout = m.x16_layout(0)
    assert layout == (1 if fmt == "q4cp" else 2)
    y0 = m.forward(0, xg).cpu().numpy()
    x16 = capi.f32_to_f16(xg, layout=layout)
    for aside in (1, 0):
        m.set_option(capi.OPT_SHARED_ASIDE, aside)
        y1 = m.forward_x16(0, xg, x16).cpu().numpy()
        assert (y1 == y0).all(), aside
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    assert max_abs_rel(y0, yo) <= TOL_LAYER
    with pytest.raises(capi.MoeError):
        m.forward_x16(0, xg[:8].contiguous(), x16[:8].contiguous())
    m.close()


@pytest.mark.parametrize("tgu,tdn,tsh,d,mid,T", [(13, 8, 12, 512, 256, 150), (12, 7, 12, 512, 256, 70), (13, 7, 8, 768, 256, 333),
                                                  (23, 20, 12, 512, 256, 90), (20, 23, 23, 256, 256, 40), (8, 8, 8, 512, 64, 100),
                                                  (13, 8, 12, 3072, 768, 200), (13, 8, 8, 3072, 768, 300), (13, 13, 13, 512, 256, 130),
                                                  (13, 12, 13, 768, 512, 260), (8, 12, 13, 512, 256, 97), (8, 7, 8, 320, 64, 50),
                                                  (7, 7, 7, 512, 256, 140), (13, 7, 7, 3072, 768, 300),
                                                  (20, 20, 20, 768, 256, 170), (23, 23, 23, 3072, 768, 200), (23, 20, 23, 512, 512, 77)])
def test_batch_layer_other_gguf_types(oracle, tgu, tdn, tsh, d, mid, T):
    """GGUF layers whose tensors are not Q4_K throughout (the reference checkpoints' Q5_K gate/up with Q5_1 / Q8_0
    down, IQ4 types, a Q8_0 MTP sidecar; src/gpu/parts/26_kernels_moe_gguf.inc:81-386): Q4_K / Q5_K gate/up and Q4_K down
    tensors on the tuned grouped GEMM, the rest on the general one, routed and shared experts in launches of their own
    where the kernels differ.  Ids bit-exact, output within the batch tolerance; the caller's f16 copy as well."""
    import torch
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(tgu * 100 + tdn + T)
    E, k = 8, 3
    hl = HostLayer(rng, d, mid, E, k, fmt="q4k", gg_types=(tgu, tdn, tsh))
    x = S.bf16_round(rng.standard_normal((T, d), dtype=np.float32))
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    xg = gpu(x)
    y = m.forward(0, xg).cpu().numpy()
    ids, _ = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    err = max_abs_rel(y, yo)
    assert err <= TOL_LAYER, err
    tuned = d % 256 == 0 and mid % 256 == 0 and (tgu in (12, 13) or tsh in (12, 13))
    assert m.x16_layout(0) == (2 if tuned else 0)
    y2 = m.forward_x16(0, xg, capi.f32_to_f16(xg, layout=m.x16_layout(0))).cpu().numpy()
    assert (y2 == y).all()
    m.set_option(capi.OPT_SHARED_ASIDE, 0)
    y3 = m.forward(0, xg).cpu().numpy()
    assert max_abs_rel(y3, yo) <= TOL_LAYER
    m.close()


@pytest.mark.gpu
@pytest.mark.parametrize("fmt,kind", [("q4cp", "bf16"), ("q4cp", "q8g64"), ("q4cp", "f32"), ("q4cp", "q8g32"), ("q4k", "bf16"),
                                      ("gg", "q8g64"), ("q4k", "q8g32")])
def test_batch_layer_with_a_densely_stored_shared_expert(oracle, fmt, kind):
    """bf16 / f32 / q8g64 / q8g32 shared-expert matrices beside q4cp, all-Q4_K and mixed-GGUF routed experts: decode, a small
    batch and a grouped-GEMM batch against the oracle (which follows the reference's matvec per storage,
    src/ref.cpp:68-109)."""
    import torch
    rng = np.random.default_rng(77)
    d, mid, E, k = 512, 256, 16, 4
    gg = (13, 8, 12) if fmt == "gg" else (12, 12, 12)
    hl = HostLayer(rng, d, mid, E, k, fmt="q4cp" if fmt == "q4cp" else "q4k", gg_types=gg, scale_std=0.02,
                   router_std=0.3, shared_dense=kind)
    m, dev = hl.to_gpu(max_tokens=300)
    L = hl.oracle_layer()
    for T in (1, 7, 32, 300):
        x = rng.standard_normal((T, d)).astype(np.float32)
        want, io, _ = oracle.moe_layer(L, x)
        y = m.forward(0, torch.from_numpy(x).cuda()).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
        assert np.abs(y - want).max() <= 2e-3 * np.abs(want).max(), (T, np.abs(y - want).max() / np.abs(want).max())
    m.close()
