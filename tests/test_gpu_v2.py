"""GPU parity of hgn v2 layers (routed experts as dtype 23 "i4r" in the Hadamard-rotated domain): bit-exact
dequantisation and rotation, the stages around the projections, the grouped GEMM with one scale per 128 columns, and
whole layers through moe_forward against the oracle (whose v2 form is pinned against the un-rotated layer in float64,
tests/test_oracle.py).  Reference: src/gpu/parts/28_kernels_hgn_v2.inc, 40_model.inc:1638-1656,4570-4686."""
import numpy as np
import pytest

from gfx1151_engine_amd import synth as S
from helpers import HostLayer, bits, max_abs_rel

pytestmark = pytest.mark.gpu
TOL_LAYER = 2e-3     # batches: f16 MFMA operands and f16 intermediates
TOL_INT = 2e-4       # small batches: integer-dot kernels (activations as four 4-bit digit planes per 32-group)


def gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.fixture(scope="module")
def capi():
    from gfx1151_engine_amd import capi as c
    c.lib()
    return c


def test_i4r_dequant_bit_exact(capi, oracle):
    rng = np.random.default_rng(61)
    rows, cols = 37, 640
    blob = S.make_i4r(rng, rows, cols, scale_std=0.02)
    sc = blob[rows * cols // 2:].view(np.float16)
    sc[:3] = [np.float16(6e-8), np.float16(0.0), np.float16(-2.5)]  # subnormal, zero, negative
    want = oracle.Mat(oracle.I4R, blob, rows, cols).dequant()
    got = capi.i4r_dequant_rows(gpu(blob), rows, cols, 0, rows).cpu().numpy()
    assert (bits(got) == bits(want)).all()
    part = capi.i4r_dequant_rows(gpu(blob), rows, cols, 5, 9).cpu().numpy()
    assert (bits(part) == bits(want[5:14])).all()


@pytest.mark.parametrize("P,n", [(1, 128), (3, 3072), (37, 768)])
def test_v2_rot_stage(capi, oracle, P, n):
    """k_v2_rot: f32 rows bit for bit (the same additions in the same order as a sequential transform), f16 rows =
    those values rounded, in the grouped GEMM's activation order; in place; without planes."""
    rng = np.random.default_rng(P + n)
    x = rng.standard_normal((P, n), dtype=np.float32)
    pre, post = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    want = oracle.v2_rot(x, pre, post)
    got = capi.v2_rot(gpu(x), gpu(pre), gpu(post)).cpu().numpy()
    assert (bits(got) == bits(want)).all()
    h = capi.from_layout1(capi.v2_rot(gpu(x), gpu(pre), None, out_f16=True)).cpu().numpy()
    assert (h == oracle.v2_rot(x, pre, None).astype(np.float16)).all()
    plain = capi.v2_rot(gpu(x)).cpu().numpy()
    assert (bits(plain) == bits(oracle.v2_rot(x))).all()
    back = capi.v2_rot(gpu(plain)).cpu().numpy()
    assert np.abs(back - x).max() <= 2e-6 * np.abs(x).max()


@pytest.mark.parametrize("mid,n", [(128, 5), (768, 23), (1024, 3), (640, 4)])
def test_i4r_mid_stage(capi, oracle, mid, n):
    """k_i4r_mid: rot_out(svh_gu) -> SwiGLU -> rot_in(suh_dn) per slot, f32 and f16 inputs / outputs."""
    rng = np.random.default_rng(mid + n)
    guv = rng.standard_normal((n, 2 * mid), dtype=np.float32) * 3
    _, svh_gu, suh_dn, _ = S.make_v2_planes(rng, 128, mid)

    def ref(z):
        z = oracle.v2_rot(z, None, svh_gu).astype(np.float64)
        g, u = z[:, :mid], z[:, mid:]
        return oracle.v2_rot((g / (1 + np.exp(-g)) * u).astype(np.float32), suh_dn, None)
    want = ref(guv)
    got = capi.i4r_mid(gpu(guv), gpu(svh_gu), gpu(suh_dn), mid).cpu().numpy()
    assert np.abs(got - want).max() <= 3e-6 * np.abs(want).max()
    g16 = guv.astype(np.float16)
    got16 = capi.from_layout1(capi.i4r_mid(gpu(g16), gpu(svh_gu), gpu(suh_dn), mid, out_f16=True)).cpu().numpy()
    want16 = ref(g16.astype(np.float32))
    assert np.abs(got16 - want16).max() <= 1e-3 * np.abs(want16).max()


@pytest.mark.parametrize("d,mid,E,k,P", [(256, 256, 6, 2, 300), (768, 512, 4, 2, 260), (3072, 768, 6, 3, 200)])
def test_i4r_grouped_gemm_stages(capi, oracle, d, mid, E, k, P):
    """moe_lut_up_raw / moe_lut_down on i4r tensors (one scale per 128 columns) and moe_v2_reduce_rot, each against
    fp64 from the oracle's dequantised rows; expert 0 left empty, tile edge cases as in the q4cp stage test."""
    from test_gpu_prefill import make_routing
    rng = np.random.default_rng(d + P + 7)
    gu = S.make_i4r(rng, E * 2 * mid, d, scale_std=0.02)
    dn = S.make_i4r(rng, E * d, mid, scale_std=0.02)
    x = rng.standard_normal((P, d), dtype=np.float32)
    ids, ws = make_routing(rng, P, E - 1, k)
    ids[:, :k] += 1
    x16 = capi.v2_rot(gpu(x), None, None, out_f16=True)  # (rotated activations in layout 1, what the launch reads)
    xr = capi.from_layout1(x16).cpu().numpy().astype(np.float64)
    r = capi.Routing(P * k, E)
    tokidx, pw, eoff, pairids = r.run(gpu(ids), gpu(ws), k)
    tiles_t, ntiles = capi.tiles(eoff, 128, P * k)
    pgu = capi.lut_i4r_view(gpu(gu), E * 2 * mid, d, 2 * mid)
    pdn = capi.lut_i4r_view(gpu(dn), E * d, mid, d)
    guv = capi.lut_up_raw(pgu, x16, tokidx, tiles_t, ntiles, mid, P * k)
    hid16 = capi.f32_to_f16(guv[:, :mid].float().contiguous())  # any f16 rows in layout 1 will do as the down input
    pairs16 = capi.lut_down(pdn, hid16, tiles_t, ntiles, d, f16=True, lut_type=capi.LUT_I4R)
    svh = S.make_v2_planes(rng, d, mid)[3]
    y = capi.v2_reduce_rot(pairs16, pairids, pw, gpu(svh), P, k).cpu().numpy()
    guv, pairs16 = guv.cpu().numpy(), pairs16.cpu().numpy()
    hid = capi.from_layout1(hid16).cpu().numpy().astype(np.float64)
    assert not np.isnan(guv).any() and not np.isnan(pairs16).any(), "every pair row must be written"
    tokidx, pw, eoff = tokidx.cpu().numpy(), pw.cpu().numpy(), eoff.cpu().numpy()
    GU = oracle.Mat(oracle.I4R, gu, E * 2 * mid, d).dequant().astype(np.float64)
    DN = oracle.Mat(oracle.I4R, dn, E * d, mid).dequant().astype(np.float64)
    acc = np.zeros((P, d))
    for e in range(E):
        sl = slice(eoff[e], eoff[e + 1])
        if sl.start == sl.stop:
            continue
        z = xr[tokidx[sl]] @ GU[e * 2 * mid:(e + 1) * 2 * mid].T
        assert np.abs(guv[sl] - z).max() <= 3e-3 * np.abs(z).max(), e
        pr = hid[sl] @ DN[e * d:(e + 1) * d].T
        assert np.abs(pairs16[sl] - pr).max() <= 3e-3 * np.abs(pr).max(), e
        np.add.at(acc, tokidx[sl], pw[sl, None].astype(np.float64) * pairs16[sl].astype(np.float64))
    want = oracle.v2_rot(acc.astype(np.float32), None, svh)
    assert np.abs(y - want).max() <= 1e-5 * np.abs(want).max()
    r.close()


def run_layer(hl, x, max_tokens=None):
    m, dev = hl.to_gpu(max_tokens=max_tokens or max(32, x.shape[0]))
    y = m.forward(0, gpu(x))
    ids, ws = m.last_routing(x.shape[0])
    out = y.cpu().numpy(), ids.cpu().numpy(), ws.cpu().numpy()
    m.close()
    return out


@pytest.mark.parametrize("d,mid,E,k,T,shared", [
    (3072, 768, 24, 10, 1, True), (3072, 768, 24, 10, 2, True), (3072, 768, 24, 10, 20, True),
    (3072, 768, 24, 10, 32, True), (256, 128, 8, 3, 5, True), (1024, 640, 8, 4, 3, True),
    (3072, 768, 24, 10, 1, False), (512, 256, 8, 2, 7, "bf16")])
def test_v2_small_batch_layer(oracle, d, mid, E, k, T, shared):
    """moe_forward on an hgn v2 layer, up to 32 tokens: q4cp shared expert in the same launches, none, or a densely
    stored one in launches of its own."""
    rng = np.random.default_rng(7000 + d + T)
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r", shared=bool(shared), shared_dense=shared if isinstance(shared, str) else None)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    y, ids, ws = run_layer(hl, x)
    assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 1e-6
    assert max_abs_rel(y, yo) <= TOL_INT, max_abs_rel(y, yo)


@pytest.mark.parametrize("d,mid,E,k,T,shared", [
    (256, 256, 6, 2, 40, True), (768, 512, 8, 4, 333, True), (3072, 768, 16, 10, 200, True),
    (512, 256, 8, 2, 150, False), (512, 256, 8, 2, 90, "q8g64"), (384, 384, 6, 2, 70, True)])
def test_v2_batch_layer(oracle, d, mid, E, k, T, shared):
    """Batches through the grouped GEMM (d, mid multiples of 256), and a shape outside it (384) that is walked through
    the small-batch path 32 rows at a time."""
    rng = np.random.default_rng(8000 + d + T)
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r", shared=bool(shared), shared_dense=shared if isinstance(shared, str) else None)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    y, ids, ws = run_layer(hl, x)
    if d % 256 == 0 and mid % 256 == 0:  # (a walked batch leaves the last 32-row chunk's ids in the context)
        assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    assert max_abs_rel(y, yo) <= TOL_LAYER, max_abs_rel(y, yo)


@pytest.mark.parametrize("d,mid,E,k,T", [(256, 256, 6, 2, 77), (768, 512, 8, 4, 333), (3072, 768, 16, 10, 200), (512, 128, 5, 1, 260)])
def test_v2_batch_middle_in_the_epilogue_equals_the_separate_launch(oracle, d, mid, E, k, T):
    """MOE_OPT_V2_FUSED_MIDDLE: the gate/up launch with the slot-wise middle in its epilogue (default) against the
    gate | up sums in memory + the middle as a launch of its own: the same arithmetic in the same order (the sums cross
    the block's waves as f16, the rounding the rows in memory have), so the layers' outputs are identical."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(8100 + d + T)
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r", shared=True)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=T)
    y1 = m.forward(0, gpu(x)).cpu().numpy()
    m.set_option(capi.OPT_V2_FUSED_MIDDLE, 0)
    y0 = m.forward(0, gpu(x)).cpu().numpy()
    m.set_option(capi.OPT_V2_FUSED_MIDDLE, 1)
    y2 = m.forward(0, gpu(x)).cpu().numpy()
    m.close()
    assert max_abs_rel(y1, yo) <= TOL_LAYER, max_abs_rel(y1, yo)
    assert (y1 == y0).all(), float(np.abs(y1 - y0).max())
    assert (y2 == y1).all()


def test_v2_layer_hc_writeback(oracle):
    """moe_forward_hc on an hgn v2 layer (the reference's k_v2_reduce_rot_hc, 28_kernels_hgn_v2.inc:189-230): the
    rotated combine written straight into the bf16 HC state, against the oracle's write-back of the oracle's y."""
    import torch
    rng = np.random.default_rng(81)
    d, mid, E, k, T = 512, 256, 8, 3, 77
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r")
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, _, _ = oracle.moe_layer(hl.oracle_layer(), x)
    w4 = rng.standard_normal((T, 4), dtype=np.float32)
    R0 = S.f32_to_bf16_bits(rng.standard_normal((T, 4, d), dtype=np.float32))
    want = oracle.hc_writeback(yo, w4, R0.copy())
    m, dev = hl.to_gpu(max_tokens=T)
    R = gpu(R0.view(np.int16))
    m.forward_hc(0, gpu(x), gpu(w4), R)
    torch.cuda.synchronize()
    got = R.cpu().numpy().view(np.uint16)
    m.close()
    a = (got.astype(np.uint32) << 16).view(np.float32)
    b = (want.astype(np.uint32) << 16).view(np.float32)
    assert np.abs(a - b).max() <= 2e-2 * np.abs(b).max()  # (one bf16 ulp of the largest state value)


@pytest.mark.parametrize("T", [1, 9, 64])
def test_v2_layer_under_graph_capture(oracle, T):
    """Decode, small batch and grouped-GEMM batch of an hgn v2 layer captured into a HIP graph and replayed with eager
    work in between; every replay equals the eager result bit for bit."""
    import torch
    rng = np.random.default_rng(82 + T)
    d, mid, E, k = 512, 256, 8, 3
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r")
    m, dev = hl.to_gpu(max_tokens=64)
    xs = [gpu(rng.standard_normal((T, d), dtype=np.float32)) for _ in range(3)]
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
    for rep in range(2):
        for i, xi in enumerate(xs):
            x.copy_(xi)
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, eager[i]), (rep, i)
            y.zero_()
            m.forward(0, xs[(i + 1) % 3], y)  # eager work between replays
            torch.cuda.synchronize()
            assert torch.equal(y, eager[(i + 1) % 3])
    m.close()


def _q6g64_blob(rng, rows, cols):
    """random q6g64 rows: codes, then (f16 scale, f16 bias) per 64 columns, row stride align16(13 cols / 16)"""
    st = (13 * cols // 16 + 15) & ~15
    blob = rng.integers(0, 256, (rows, st), dtype=np.uint8)
    sb = np.stack([rng.uniform(0.005, 0.03, (rows, cols // 64)), rng.uniform(-1, 1, (rows, cols // 64))], -1).astype(np.float16)
    blob[:, 3 * cols // 4: 3 * cols // 4 + cols // 64 * 4] = sb.view(np.uint8).reshape(rows, -1)
    return blob


def _planes(rng, n):
    return (rng.uniform(0.5, 1.5, n) * rng.choice([-1, 1], n)).astype(np.float16).astype(np.float32)


def test_v2_dense_tensors_to_bf16_bit_exact(capi, oracle):
    """ht (dtype 16) and q6g64 (dtype 24) -> the bf16 matrix of the reference's v2_deq_bf16, bit for bit against the
    oracle (ht: random code streams -- every stream is a valid tensor --, several tiles both ways, signed planes)."""
    rng = np.random.default_rng(71)
    for rows, cols in ((128, 128), (256, 384), (384, 1024)):
        codes = rng.integers(0, 256, rows * cols // 2, dtype=np.uint8)
        suh, svh = _planes(rng, cols), _planes(rng, rows)
        want = oracle.v2_dense_bf16(16, codes, rows, cols, suh, svh)
        got = capi.v2_dense_to_bf16(capi.HT, gpu(codes), rows, cols, gpu(suh), gpu(svh)).cpu().numpy().view(np.uint16)
        assert (got == want).all(), (rows, cols)
    for rows, cols in ((1, 256), (5, 192), (130, 3072)):
        blob = _q6g64_blob(rng, rows, cols)
        want = oracle.v2_dense_bf16(24, blob, rows, cols)
        got = capi.v2_dense_to_bf16(capi.Q6G64, gpu(blob), rows, cols).cpu().numpy().view(np.uint16)
        assert (got == want).all(), (rows, cols)
    # shapes off the grid, a missing plane, another dtype
    import torch
    out = torch.empty(128 * 128, dtype=torch.int16, device="cuda")
    c = gpu(np.zeros(128 * 128, np.uint8))
    f = gpu(np.ones(128, np.float32))
    L = capi.lib()
    u64 = capi.u64
    assert L.moe_v2_dense_to_bf16(16, capi.ptr(c), capi.ptr(f), capi.ptr(f), u64(64), u64(128), capi.ptr(out), capi.stream()) == -2
    assert L.moe_v2_dense_to_bf16(16, capi.ptr(c), None, capi.ptr(f), u64(128), u64(128), capi.ptr(out), capi.stream()) == -2
    assert L.moe_v2_dense_to_bf16(24, capi.ptr(c), None, None, u64(4), u64(96), capi.ptr(out), capi.stream()) == -2
    assert L.moe_v2_dense_to_bf16(5, capi.ptr(c), None, None, u64(128), u64(128), capi.ptr(out), capi.stream()) == -1
