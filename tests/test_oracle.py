"""CPU-only: pins the oracle (oracle/moe_oracle.c) against
 (1) golden vectors produced by the reference's own code (tests/golden/*.npz),
 (2) the reference's own code directly where oracle/_ref is built (this container),
 (3) closed forms, invariants and brute force that a dropped term / wrong index would break."""
import numpy as np
import pytest

from gfx1151_engine_amd import synth as S
from helpers import HostLayer, bits


def same_bits(a, b):
    a, b = bits(a), np.asarray(b, np.uint32)
    nan = (np.isnan(a.view(np.float32)) & np.isnan(b.view(np.float32)))
    return bool(((a == b) | nan).all())


# ---------- fp16 ----------
def test_fp16_all_patterns_golden(oracle, golden):
    want = golden("fp16_table.npz")["bits"]
    got = np.array([oracle.fp16_to_f32(h) for h in range(65536)], np.float32)
    assert same_bits(got, want)


def test_fp16_matches_numpy(oracle):
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([oracle.fp16_to_f32(int(x)) for x in h], np.float32)
    ok = np.isfinite(want)
    assert (bits(got[ok]) == bits(want[ok])).all()


# ---------- q4cp ----------
def test_q4cp_golden(oracle, golden):
    g = golden("q4cp_rows.npz")
    for i in range(int(g["n"])):
        rows, cols = (int(v) for v in g[f"shape{i}"])
        got = oracle.q4cp_rows(g[f"blob{i}"], rows, cols, 0, rows)
        assert same_bits(got, g[f"bits{i}"]), f"case {i}"


def test_q4cp_layout_closed_form(oracle):
    """Independent numpy decode of the byte layout: codebook, low nibble first, padded scale record."""
    rng = np.random.default_rng(5)
    rows, cols = 7, 640
    cb = rng.uniform(-2, 2, 16).astype(np.float32)
    blob = S.make_q4cp(rng, rows, cols, codebook=cb, scale_std=0.5)
    ss = 48  # 40 B of scales padded to 16 B
    assert S.q4cp_scale_stride(cols) == ss == oracle.lib().orc_q4cp_scale_stride(cols)
    assert blob.size == 64 + rows * cols // 2 + rows * ss == oracle.lib().orc_q4cp_blob_bytes(rows, cols)
    codes = blob[64:64 + rows * cols // 2].reshape(rows, cols // 2)
    nib = np.stack([codes & 0xF, codes >> 4], axis=-1).reshape(rows, cols)
    sc = blob[64 + rows * cols // 2:].reshape(rows, ss)[:, :cols // 16].copy().view(np.float16).astype(np.float32)
    want = cb[nib] * np.repeat(sc, 32, axis=1)
    assert same_bits(oracle.q4cp_rows(blob, rows, cols, 0, rows), bits(want))
    # row offset argument
    assert same_bits(oracle.q4cp_rows(blob, rows, cols, 3, 2), bits(want[3:5]))


def test_q4cp_vs_reference_build(oracle):
    if oracle.ref() is None:
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(11)
    for rows, cols in [(9, 640), (3, 3072), (16, 32)]:
        blob = S.make_q4cp(rng, rows, cols, codebook=rng.standard_normal(16).astype(np.float32), scale_std=1.0)
        assert same_bits(oracle.q4cp_rows(blob, rows, cols, 0, rows),
                         bits(oracle.ref_q4cp_rows(blob, rows, cols, 0, rows)))


# ---------- Q4_K ----------
def test_q4k_golden(oracle, golden):
    g = golden("q4k_rows.npz")
    for i in range(int(g["n"])):
        rows, cols = (int(v) for v in g[f"shape{i}"])
        assert same_bits(oracle.q4k_rows(g[f"raw{i}"], rows, cols), g[f"bits{i}"]), f"case {i}"
    for i in range(g["k4_q"].shape[0]):
        for j in range(8):
            assert oracle.scale_min_k4(j, g["k4_q"][i]) == tuple(int(v) for v in g["k4_sm"][i, j])


def test_q4k_scale_pack_roundtrip_bruteforce(oracle):
    """All 64 x 64 (scale, min) values in every one of the 8 positions survive pack -> unpack."""
    vals = np.arange(64, dtype=np.uint8)
    for j in range(8):
        for m in (0, 21, 63):
            sc = np.zeros((64, 8), np.uint8)
            mn = np.full((64, 8), m, np.uint8)
            sc[:, j] = vals
            q = S.pack_scale_min_k4(sc, mn)
            for v in range(64):
                assert oracle.scale_min_k4(j, q[v]) == (v, m)
            q = S.pack_scale_min_k4(mn, sc)
            for v in range(64):
                assert oracle.scale_min_k4(j, q[v]) == (m, v)


def test_q4k_closed_form(oracle):
    """y = d*sc*q - dmin*m with the documented element order (low nibbles then high nibbles of 32 bytes)."""
    rng = np.random.default_rng(3)
    raw = S.make_q4k(rng, 1, 512)
    y = oracle.q4k_rows(raw, 1, 512)[0]
    for b in range(2):
        blk = raw[b * 144:(b + 1) * 144]
        d, dmin = (float(v) for v in blk[:4].copy().view(np.float16).astype(np.float32))
        for j in range(4):
            s0, m0 = oracle.scale_min_k4(2 * j, blk[4:16])
            s1, m1 = oracle.scale_min_k4(2 * j + 1, blk[4:16])
            qs = blk[16 + 32 * j:16 + 32 * j + 32]
            lo = np.float32(d * s0) * (qs & 0xF).astype(np.float32) - np.float32(dmin * m0)
            hi = np.float32(d * s1) * (qs >> 4).astype(np.float32) - np.float32(dmin * m1)
            got = y[b * 256 + 64 * j: b * 256 + 64 * j + 64]
            assert same_bits(got[:32], bits(lo)) and same_bits(got[32:], bits(hi))


def test_q4k_vs_reference_build(oracle):
    if oracle.ref() is None:
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(12)
    raw = S.make_q4k(rng, 5, 1024, scale_std=1.0)
    assert same_bits(oracle.q4k_rows(raw, 5, 1024), bits(oracle.ref_q4k_rows(raw, 5, 1024)))
    assert oracle.lib().orc_q4k_row_bytes(3072) == oracle.ref().ref_q4k_row_bytes(3072) == 1728


# ---------- router ----------
def test_router_matches_float64_numpy(oracle):
    rng = np.random.default_rng(21)
    E, d, k, T = 64, 96, 10, 9
    W = rng.standard_normal((E, d)).astype(np.float32) * 0.3
    x = rng.standard_normal((T, d)).astype(np.float32)
    logits, ids, ws = oracle.router(oracle.Mat(oracle.F32, W, E, d), x, k)
    # sequential fp64 accumulation == math.fsum to within the last f32 bit; check exact order on a small case
    for t in range(T):
        for e in range(0, E, 7):
            acc = 0.0
            for c in range(d):
                acc += float(W[e, c]) * float(x[t, c])
            assert np.float32(acc) == logits[t, e]
        p = np.exp(logits[t].astype(np.float64) - logits[t].max())
        p = (p.astype(np.float32).astype(np.float64) / p.astype(np.float32).astype(np.float64).sum()).astype(np.float32)
        order = np.lexsort((np.arange(E), -p))[:k]  # value desc, index asc
        assert (ids[t, :k] == order).all()
        w = (p[order].astype(np.float64) / p[order].astype(np.float64).sum()).astype(np.float32)
        assert (bits(ws[t, :k]) == bits(w)).all()
        assert abs(float(ws[t, :k].sum()) - 1.0) < 1e-6 and len(set(ids[t, :k])) == k


def test_router_f32_equals_bf16_on_representable_weights(oracle):
    """f32 router rows (no f32 branch in the reference's matvec) reduce to the bf16 branch, which the
    reference build pins, when every weight is bf16-representable."""
    rng = np.random.default_rng(12)
    T, E, d, k = 3, 24, 96, 5
    Wb = S.f32_to_bf16_bits((rng.standard_normal((E, d)) * 0.3).astype(np.float32))
    Wf = (Wb.astype(np.uint32) << 16).view(np.float32)
    x = rng.standard_normal((T, d)).astype(np.float32)
    la, ia, wa = oracle.router(oracle.Mat(oracle.F32, Wf, E, d), x, k)
    lb, ib, wb = oracle.router(oracle.Mat(oracle.BF16, Wb, E, d), x, k)
    assert (bits(la) == bits(lb)).all() and (ia == ib).all() and (bits(wa) == bits(wb)).all()


def test_router_ties_and_special_cases(oracle):
    E, k = 32, 5
    # uniform logits: every probability equal -> lowest indices, equal weights
    p, ids, ws = oracle.softmax_topk(np.zeros(E, np.float32), k)
    assert list(ids) == [0, 1, 2, 3, 4] and np.allclose(ws, 0.2) and np.allclose(p, 1.0 / E)
    # one-hot: that expert first with weight ~1, the rest tie -> lowest indices
    lg = np.zeros(E, np.float32)
    lg[17] = 30.0
    p, ids, ws = oracle.softmax_topk(lg, k)
    assert list(ids) == [17, 0, 1, 2, 3] and ws[0] > 0.999
    # k == E returns a permutation sorted by logit
    lg = np.random.default_rng(2).standard_normal(E).astype(np.float32)
    p, ids, ws = oracle.softmax_topk(lg, E)
    assert (np.diff(lg[ids]) <= 0).all() and sorted(ids) == list(range(E))
    # pairs of equal logits: lower index wins
    lg = np.repeat(np.arange(16, dtype=np.float32), 2)[::-1].copy()
    p, ids, ws = oracle.softmax_topk(lg, 6)
    assert list(ids) == [0, 1, 2, 3, 4, 5]


# ---------- permutation ----------
def test_route_invariants_and_bruteforce(oracle):
    rng = np.random.default_rng(31)
    P, E, k = 300, 40, 6
    ids = np.zeros((P, 16), np.int32)
    ws = np.zeros((P, 16), np.float32)
    for t in range(P):
        ids[t, :k] = rng.choice(E - 3, k, replace=False)  # experts E-3.. stay empty
        ws[t, :k] = rng.random(k)
    tokidx, pw, eoff, pairids = oracle.route(ids, ws, k, E)
    assert eoff[0] == 0 and eoff[E] == P * k and (np.diff(eoff) >= 0).all()
    flat = [(ids[t, s], t * k + s) for t in range(P) for s in range(k)]
    order = sorted(flat)  # stable sort by (expert, original pair index)
    for q, (e, p0) in enumerate(order):
        t, s = divmod(p0, k)
        assert tokidx[q] == t and pw[q] == ws[t, s] and eoff[e] <= q < eoff[e + 1]
    assert sorted(pairids) == list(range(P * k))
    for t in range(0, P, 17):
        es = [ids[t, s] for s in range(k)]
        for rank, e in enumerate(sorted(es)):
            q = pairids[t * k + rank]
            assert tokidx[q] == t and eoff[e] <= q < eoff[e + 1]
    tl = oracle.tiles(eoff, 64)
    assert tl[:, 2].sum() == P * k and (tl[:, 2] <= 64).all() and (tl[:, 2] > 0).all()
    assert (np.diff(tl[:, 0]) >= 0).all()


# ---------- the layer ----------
def test_layer_golden_from_reference_moe(oracle, golden):
    """Model::moe of the reference (src/ref.cpp:563-637) on tiny synthetic checkpoints: bit-identical y."""
    g = golden("moe_layer.npz")
    for i in range(int(g["n"])):
        d, mid, E, k, sh_dt = (int(v) for v in g[f"cfg{i}"])
        O = oracle
        sh = [O.Mat(sh_dt, g[f"shg{i}"], mid, d), O.Mat(sh_dt, g[f"shu{i}"], mid, d),
              O.Mat(sh_dt, g[f"shd{i}"], d, mid), O.Mat(O.BF16, g[f"sg{i}"], 1, d)]
        L = O.Layer(d, mid, E, k, O.Mat(O.BF16, g[f"router{i}"], E, d), O.Mat(O.Q4CP, g[f"dn{i}"], E * d, mid),
                    gate_up=O.Mat(O.Q4CP, g[f"gu{i}"], E * 2 * mid, d), shared=sh)
        y, ids, ws = O.moe_layer(L, g[f"x{i}"])
        assert (bits(y) == g[f"ybits{i}"]).all(), f"case {i}"
        # token subset path gives the same rows
        y2, _, _ = O.moe_layer(L, g[f"x{i}"], tok_list=[4, 1])
        assert (bits(y2[[1, 4]]) == g[f"ybits{i}"][[1, 4]]).all() and np.isnan(y2[0]).all()


def test_q8g64_dequant_golden(oracle, golden):
    """Checkpoint::dequant of the reference on a q8g64 tensor (src/hgn.h:189-202): bit-identical rows."""
    g = golden("moe_layer.npz")
    m = oracle.Mat(oracle.Q8G64, g["q8g64_raw"], 5, 192)
    assert (bits(m.dequant()) == g["q8g64_bits"]).all()
    assert (bits(m.dequant(2, 2)) == g["q8g64_bits"][2:4]).all()
    # closed form on hand-made bytes: code * scale + min
    raw = np.zeros((1, 64 + 4), np.uint8)
    raw[0, :64] = np.arange(64) * 4
    raw[0, 64:].view(np.float16)[:] = [0.5, -3.0]
    w = oracle.Mat(oracle.Q8G64, raw, 1, 64).dequant()
    assert (w[0] == np.arange(64, dtype=np.float32) * 4 * 0.5 - 3.0).all()


def test_q8g32_dequant_golden(oracle, golden):
    """Checkpoint::dequant of the reference on a planar q8g32 tensor (src/hgn.h:176-183): bit-identical rows, from
    the committed vector and (where the reference build is present) live on another tensor.  The reference's CPU
    matvec has no q8g32 branch (src/ref.cpp:68-109 throws for it), so a layer with such a shared expert is the
    dequantised row in the generic fp64 dot product: that form is not pinned by a run of the reference."""
    g = golden("moe_layer.npz")
    m = oracle.Mat(oracle.Q8G32, g["q8g32_raw"], 6, 96)
    assert (bits(m.dequant()) == g["q8g32_bits"]).all()
    assert (bits(m.dequant(4, 2)) == g["q8g32_bits"][4:6]).all()
    raw = np.zeros(64 + 4, np.uint8)  # two rows of 32: codes -128..127 step 4, scales 0.25 and -2
    raw[:64] = (np.arange(64) * 4 - 128).astype(np.int8).view(np.uint8)
    raw[64:].view(np.float16)[:] = [0.25, -2.0]
    w = oracle.Mat(oracle.Q8G32, raw, 2, 32).dequant()
    assert (w[0] == (np.arange(32) * 4 - 128) * 0.25).all() and (w[1] == (np.arange(32, 64) * 4 - 128) * -2.0).all()
    if oracle.ref() is not None:
        rng = np.random.default_rng(9)
        q = S.quantize_q8g32(rng.standard_normal((8, 160)).astype(np.float32))
        mm = oracle.Mat(oracle.Q8G32, q, 8, 160)
        assert (bits(mm.dequant()) == bits(oracle.ref_dequant_tensor(mm))).all()


def test_q8g64_shared_expert_vs_reference_build(oracle):
    """The reference's q8g64 matvec sums per 64-group (code . x) * scale + min * sum(x) (src/ref.cpp:91-106), not the
    dot with the dequantised row: the oracle follows it to the bit."""
    if oracle.ref() is None:
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(43)
    d, mid, E, k = 192, 128, 6, 2
    hl = HostLayer(rng, d, mid, E, k, router_dtype="bf16", scale_std=0.05, router_std=0.3, shared_dense="q8g64")
    L = hl.oracle_layer()
    L.shared[3] = oracle.Mat(oracle.BF16, S.f32_to_bf16_bits(hl.shared[3]), 1, d)
    x = rng.standard_normal((3, d)).astype(np.float32)
    y, ids, ws = oracle.moe_layer(L, x)
    for t in range(3):
        assert (bits(oracle.ref_moe_token(L, x[t])) == bits(y[t])).all()


def test_layer_vs_reference_build_random(oracle):
    if oracle.ref() is None:
        pytest.skip("oracle/_ref not built here")
    rng = np.random.default_rng(41)
    d, mid, E, k = 160, 96, 10, 4
    hl = HostLayer(rng, d, mid, E, k, router_dtype="bf16", scale_std=0.05, router_std=0.3)
    L = hl.oracle_layer()
    # the reference's matvec has no f32 branch: give it the shared gate as bf16 (same values)
    sg16 = S.f32_to_bf16_bits(hl.shared[3])
    L.shared[3] = oracle.Mat(oracle.BF16, sg16, 1, d)
    x = rng.standard_normal((3, d)).astype(np.float32)
    y, ids, ws = oracle.moe_layer(L, x)
    for t in range(3):
        assert (bits(oracle.ref_moe_token(L, x[t])) == bits(y[t])).all()


def test_layer_textbook_special_cases(oracle):
    """Identity-like weights: one expert, codebook value 1 on the diagonal groups -> hand-computable."""
    O = oracle
    d = mid = 32
    E, k = 2, 1
    cb = np.zeros(16, np.float32)
    cb[1] = 1.0
    # expert 0: gate row r = e_r (code 1 at column r), up the same, down identity; expert 1: zeros
    def eye_codes(rows):
        c = np.zeros((rows, 16), np.uint8)
        for r in range(rows):
            col = r % 32
            c[r, col // 2] = 1 << (4 * (col % 2))
        return c
    gu_codes = np.zeros((E * 2 * mid, 16), np.uint8)
    gu_codes[:2 * mid] = eye_codes(2 * mid)
    dn_codes = np.zeros((E * d, 16), np.uint8)
    dn_codes[:d] = eye_codes(d)
    one = np.ones((E * 2 * mid, 1), np.float16)
    gu = S.make_q4cp(None, E * 2 * mid, d, codebook=cb, scales=one, codes=gu_codes)
    dn = S.make_q4cp(None, E * d, mid, codebook=cb, scales=np.ones((E * d, 1), np.float16), codes=dn_codes)
    Wr = np.zeros((E, d), np.float32)
    Wr[0, 0] = 50.0  # x[0] > 0 -> expert 0
    L = O.Layer(d, mid, E, k, O.Mat(O.F32, Wr, E, d), O.Mat(O.Q4CP, dn, E * d, mid),
                gate_up=O.Mat(O.Q4CP, gu, E * 2 * mid, d))
    x = np.linspace(0.5, 2.0, d, dtype=np.float32)[None]
    y, ids, ws = O.moe_layer(L, x)
    assert ids[0, 0] == 0 and ws[0, 0] == 1.0
    want = (x[0] / (1 + np.exp(-x[0].astype(np.float64)))).astype(np.float32) * x[0]  # silu(x)*x
    assert np.allclose(y[0], want, rtol=1e-6)
    # zero activations: silu(0)*0 = 0 everywhere
    y0, _, _ = O.moe_layer(L, np.zeros((1, d), np.float32))
    assert (y0 == 0).all()


def test_layer_matches_float64_numpy_q4k(oracle):
    """Q4_K layer against an independent numpy float64 evaluation from the dequantised matrices."""
    O = oracle
    rng = np.random.default_rng(51)
    d, mid, E, k = 256, 256, 6, 3
    hl = HostLayer(rng, d, mid, E, k, fmt="q4k", scale_std=0.02, router_std=0.2)
    L = hl.oracle_layer()
    x = rng.standard_normal((4, d)).astype(np.float32)
    y, ids, ws = O.moe_layer(L, x)
    G, U, D = L.gate.dequant().astype(np.float64), L.up.dequant().astype(np.float64), L.down.dequant().astype(np.float64)
    shg, shu, shd, sg = (m.dequant().astype(np.float64) for m in L.shared)
    for t in range(4):
        xt = x[t].astype(np.float64)
        acc = np.zeros(d)
        for s in range(k):
            e = ids[t, s]
            g = G[e * mid:(e + 1) * mid] @ xt
            u = U[e * mid:(e + 1) * mid] @ xt
            h = g / (1 + np.exp(-g)) * u
            acc += float(ws[t, s]) * (D[e * d:(e + 1) * d] @ h)
        g, u = shg @ xt, shu @ xt
        ey = shd @ (g / (1 + np.exp(-g)) * u)
        want = acc + ey / (1 + np.exp(-(sg @ xt)))
        assert np.abs(y[t] - want).max() <= 2e-5 * np.abs(want).max()


def test_i4r_rows_closed_form(oracle):
    """hgn v2 i4r rows: every code value times positive, negative, subnormal and zero scales against the published
    layout evaluated element-wise in numpy (codes plane, low nibble first, then one fp16 scale per 128 columns, rows
    unpadded; w = (n - 8) * scale, exact in f32)."""
    O = oracle
    rows, cols = 6, 384
    rng = np.random.default_rng(23)
    codes = rng.integers(0, 256, size=(rows, cols // 2), dtype=np.uint8)
    codes[0, :8] = [0x10, 0x32, 0x54, 0x76, 0x98, 0xBA, 0xDC, 0xFE]  # elements 0..15 of row 0 hold the codes 0..15
    sc = (rng.standard_normal((rows, cols // 128)) * 0.02).astype(np.float16)
    sc[1, 0], sc[2, 1], sc[3, 2] = np.float16(6e-8), np.float16(0.0), np.float16(-1.5)
    blob = np.concatenate([codes.reshape(-1), sc.reshape(-1).view(np.uint8)])
    got = O.Mat(O.I4R, blob, rows, cols).dequant()
    q = np.stack([codes & 15, codes >> 4], -1).reshape(rows, cols).astype(np.float32) - 8
    want = (q.reshape(rows, -1, 128) * sc.astype(np.float32)[..., None]).reshape(rows, cols)
    assert same_bits(got, bits(want))
    assert (got[0, :16] == (np.arange(16, dtype=np.float32) - 8) * np.float32(sc[0, 0])).all()


def test_v2_rotation_against_the_hadamard_matrix(oracle):
    """rot(x) = post * H(pre * x) / sqrt(128) per 128 block against scipy's Sylvester matrix in float64; H / sqrt(128) is
    its own inverse; a unit vector gives a column of +-1 / sqrt(128) with the sign pattern popcount(i & j)."""
    from scipy.linalg import hadamard
    O = oracle
    rng = np.random.default_rng(24)
    n = 384
    x = rng.standard_normal((5, n)).astype(np.float32)
    pre, post = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    Hn = hadamard(128).astype(np.float64) / np.sqrt(128.0)
    want = np.stack([np.concatenate([Hn @ (x[t, b:b + 128].astype(np.float64) * pre[b:b + 128]) for b in range(0, n, 128)])
                     for t in range(5)]) * post
    got = O.v2_rot(x, pre, post)
    assert np.abs(got - want).max() <= 2e-6 * np.abs(want).max()
    back = O.v2_rot(O.v2_rot(x))
    assert np.abs(back - x).max() <= 2e-6 * np.abs(x).max()
    e = np.zeros((1, 128), np.float32)
    e[0, 77] = 1.0
    col = O.v2_rot(e)[0]
    sign = np.array([(-1) ** bin(i & 77).count("1") for i in range(128)], np.float32)
    assert (col == sign * np.float32(0.0883883476483184405)).all()


def test_v2_layer_equals_the_unrotated_layer_in_float64(oracle):
    """An hgn v2 layer (rotated i4r experts) against an independent float64 evaluation of the ordinary layer on the
    un-rotated weights W = diag(svh) . Hn . G . Hn . diag(suh) (Hn = block-diagonal H / sqrt(128)): a wrong plane, a
    swapped input / output side or a missing rotation would change the result by O(1)."""
    from scipy.linalg import hadamard
    O = oracle
    rng = np.random.default_rng(25)
    d, mid, E, k = 256, 128, 6, 3
    hl = HostLayer(rng, d, mid, E, k, fmt="i4r", scale_std=0.02, router_std=0.2)
    L = hl.oracle_layer()
    x = rng.standard_normal((4, d)).astype(np.float32)
    y, ids, ws = O.moe_layer(L, x)
    su, svh_gu, suh_dn, svh_dn = (p.astype(np.float64) for p in hl.planes)
    Hn = hadamard(128).astype(np.float64) / np.sqrt(128.0)

    def unrot(G, sv, su_):  # G [O][K] in the rotated domain -> W
        O_, K = G.shape
        W = G.reshape(O_, K // 128, 128) @ Hn           # . Hn on the input side (Hn symmetric)
        W = W.reshape(O_, K)
        W = (Hn @ W.reshape(O_ // 128, 128, K)).reshape(O_, K)
        return sv[:, None] * W * su_[None, :]
    GU = L.gate_up.dequant().astype(np.float64)
    DN = L.down.dequant().astype(np.float64)
    shg, shu, shd, sg = (m.dequant().astype(np.float64) for m in L.shared)
    for t in range(4):
        xt = x[t].astype(np.float64)
        acc = np.zeros(d)
        for s in range(k):
            e = ids[t, s]
            W = unrot(GU[e * 2 * mid:(e + 1) * 2 * mid], svh_gu, su)
            g, u = W[:mid] @ xt, W[mid:] @ xt
            h = g / (1 + np.exp(-g)) * u
            acc += float(ws[t, s]) * (unrot(DN[e * d:(e + 1) * d], svh_dn, suh_dn) @ h)
        g, u = shg @ xt, shu @ xt
        want = acc + (shd @ (g / (1 + np.exp(-g)) * u)) / (1 + np.exp(-(sg @ xt)))
        assert np.abs(y[t] - want).max() <= 2e-5 * np.abs(want).max()


@pytest.mark.parametrize("t,name", [(13, "Q5_K"), (8, "Q8_0"), (7, "Q5_1"), (12, "Q4_K"), (20, "IQ4_NL"), (23, "IQ4_XS")])
def test_gg_rows_against_reference(oracle, t, name):
    """The further ggml block types of the expert tensors: the oracle's rows against the reference's own
    gguf::dequant_row (oracle/_ref) on random block bytes, bit for bit, and against a numpy evaluation of the
    published block layout for one type with every code value present (Q8_0: d * int8)."""
    O = oracle
    rng = np.random.default_rng(t)
    rows, cols = 5, 768
    raw = S.make_gg(rng, t, rows, cols)
    got = O.gg_rows(t, raw, rows, cols)
    assert np.isfinite(got).all()
    if O.ref() is not None:
        assert O.gg_row_bytes(t, cols) == int(O.ref().ref_gg_row_bytes(t, cols))
        want = O.ref_gg_rows(t, raw, rows, cols)
        assert (got.view(np.uint32) == want.view(np.uint32)).all(), name
    if t == 8:
        blk = raw.reshape(-1, 34)
        d = blk[:, :2].copy().view(np.float16).astype(np.float32)
        q = blk[:, 2:].copy().view(np.int8).astype(np.float32)
        assert ((d * q).reshape(rows, cols).view(np.uint32) == got.view(np.uint32)).all()
    if t == 7:
        blk = raw.reshape(-1, 24)
        d = blk[:, :2].copy().view(np.float16).astype(np.float32)
        m = blk[:, 2:4].copy().view(np.float16).astype(np.float32)
        qh = blk[:, 4:8].copy().view(np.uint32)
        qs = blk[:, 8:]
        j = np.arange(16)
        x0 = (qs & 15) | (((qh >> j) & 1) << 4)
        x1 = (qs >> 4) | (((qh >> (j + 16)) & 1) << 4)
        y = np.concatenate([x0, x1], 1).astype(np.float32) * d + m
        assert (y.reshape(rows, cols).view(np.uint32) == got.view(np.uint32)).all()


def test_hc_writeback_closed_forms(oracle):
    """HC write-back of the combine (src/gpu/parts/24_kernels_moe_lt.inc:126-161).  Cases that the formula fixes
    without retyping it: gate logit 0 gives inj = 1 exactly, so R' = bf16(R + y) (checked against an independent
    round-to-nearest-even through float64 arithmetic on values where the sum is exact in f32); a very negative logit
    gives inj = 0 and leaves R as it is; a very positive one gives inj = 2; halfway cases round to even."""
    O = oracle
    rng = np.random.default_rng(4)
    P, D = 3, 64
    # small integers: every R + y below is exact in f32 and in f64
    y = rng.integers(-200, 200, (P, D)).astype(np.float32)
    Rf = rng.integers(-100, 100, (P, 4, D)).astype(np.float32)
    R = (Rf.view(np.uint32) >> 16).astype(np.uint16)  # small integers are exact in bf16
    w4 = np.zeros((P, 4), np.float32)
    w4[:, 1] = -1e4   # inj = 2 / (1 + inf) = 0
    w4[:, 2] = 1e4    # inj = 2 / (1 + 0) = 2
    got = O.hc_writeback(y, w4, R)

    def bf16_rne(a64):  # independent: nearest bf16 of exactly representable reals, ties to even
        a = a64.astype(np.float32)
        u = a.view(np.uint32).astype(np.uint64)
        low = u & 0xFFFF
        up = u >> 16
        rnd = (low > 0x8000) | ((low == 0x8000) & ((up & 1) == 1))
        return (up + rnd).astype(np.uint16)
    assert (got[:, 0] == bf16_rne(Rf[:, 0].astype(np.float64) + y)).all()
    assert (got[:, 3] == bf16_rne(Rf[:, 3].astype(np.float64) + y)).all()
    assert (got[:, 1] == R[:, 1]).all()
    assert (got[:, 2] == bf16_rne(Rf[:, 2].astype(np.float64) + 2.0 * y)).all()
    # ties: 257 = 0x1.01p8 lies halfway between the bf16 neighbours 256 and 258 -> 256 (even); 259 -> 260
    y2 = np.array([[1.0, 3.0]], np.float32)
    R2 = np.zeros((1, 4, 2), np.uint16)
    R2[:] = (np.float32(256.0).view(np.uint32) >> 16).astype(np.uint16)
    out = O.hc_writeback(y2, np.zeros((1, 4), np.float32), R2)
    vals = (out.astype(np.uint32) << 16).view(np.float32)
    assert (vals[0, :, 0] == 256.0).all() and (vals[0, :, 1] == 260.0).all()
    # a gate strictly between the saturated ends: w4 = 4 ln 3 gives inj = 2 / (1 + 1/3) = 1.5 (to within an ulp of
    # the f32 exp), w4 = -4 ln 3 gives 2 / (1 + 3) = 0.5.  With R = 0 and y = 2^j the results 1.5 * 2^j and 0.5 * 2^j
    # are bf16 numbers that an ulp of inj cannot move; a wrong divisor in inj (w4 / 2, w4 / 8) or a missing factor 2
    # gives 1.8 / 1.27 / 0.75 times y instead and fails.
    y3 = np.array([[2.0, -4.0, 0.5, 64.0]], np.float32)
    w3 = np.array([[4 * np.log(3.0), -4 * np.log(3.0), 4 * np.log(7.0), 0.0]], np.float32)  # inj 1.5, 0.5, 1.75, 1
    out3 = O.hc_writeback(y3, w3, np.zeros((1, 4, 4), np.uint16))
    v3 = (out3.astype(np.uint32) << 16).view(np.float32)
    for b, inj in enumerate((1.5, 0.5, 1.75, 1.0)):
        assert (v3[0, b] == inj * y3[0]).all(), (b, v3[0, b])


# ---------- hgn v2 dense tensors: ht (dtype 16), q6g64 (dtype 24) ----------
def _bf16_to_f64(b):
    return (np.asarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32).astype(np.float64)


def test_ht_alphabet(oracle):
    """The 65536 values of the hashed alphabet.  w16 = 0 hashes to byte sum 0: 1024 * 1.732421875 / 256 - 10.3828125 =
    -3.453125, exact in f16.  The byte sum of a well-mixed 32-bit word is the sum of four uniform bytes (mean 510,
    variance 4 * (256^2 - 1) / 12), so the alphabet is a unit normal's: mean -0.0017, standard deviation 1.0003 -- which
    fixes both constants.  Every value is an f16, rounded as numpy rounds f32 to f16 (the oracle converts by hand)."""
    v = np.array([oracle.ht_value(i) for i in range(65536)], np.float32)
    assert v[0] == np.float32(-3.453125)
    assert abs(float(v.mean()) + 0.0017) < 5e-3 and abs(float(v.std()) - 1.0003) < 5e-3
    assert (v.astype(np.float16).astype(np.float32) == v).all()
    w = np.arange(65536, dtype=np.uint64)
    t = (w * np.uint64(0x83DCD12D)) & np.uint64(0xFFFFFFFF)
    s = (t & 0xFF) + ((t >> 8) & 0xFF) + ((t >> 16) & 0xFF) + (t >> 24)
    exact = (1024 + s).astype(np.float64) * float(np.float32(1.732421875 / 256)) + (-10.3828125)  # exact in float64
    assert (np.float32(exact).astype(np.float16).astype(np.float32) == v).all()


def test_ht_decode_against_the_reference_encoder(oracle, tmp_path):
    """The reference's own ht encoder (tools/v2repro/htenc.cc, built as oracle/_ref/htenc) searches the code stream whose
    decoded values are nearest to a target, in the official tile layout, and prints the mean squared error it reached.
    Decoding its stream here must give that same error: a wrong tile / granule / row / column index, a window taken from
    the wrong bits or the wrong neighbouring word would leave the decoded values uncorrelated with the target (relative
    error 1.4 instead of 0.24)."""
    import os
    import shutil
    import subprocess
    exe = os.path.join(os.path.dirname(oracle.__file__), "_ref", "htenc")
    if not os.path.exists(exe):
        pytest.skip("oracle/_ref/htenc is not built (the reference tree is not here)")
    shutil.copy(exe, tmp_path / "htenc")  # the encoder reads ht_lut.f32 from its own directory
    np.array([oracle.ht_value(i) for i in range(65536)], np.float32).tofile(tmp_path / "ht_lut.f32")
    rng = np.random.default_rng(41)
    rows, cols = 256, 384  # 2 x 3 tiles
    G = rng.standard_normal((rows, cols)).astype(np.float32)
    G.tofile(tmp_path / "t.f32")
    r = subprocess.run([str(tmp_path / "htenc"), "t.f32", str(rows), str(cols), "o.codes", "16", "2"], cwd=tmp_path,
                       capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr
    said = float(r.stderr.split("mse")[1].split()[0])
    got = oracle.ht_decode(np.fromfile(tmp_path / "o.codes", np.uint8), rows, cols)
    mse = float(((got.astype(np.float64) - G) ** 2).mean())
    assert abs(mse - said) <= 1e-5 * said, (mse, said)
    assert mse < 0.08


def test_v2_dense_ht_is_the_unrotated_matrix(oracle):
    """bf16 W of an ht tensor = diag(svh) . H . G . H . diag(suh) / 128 (H = scipy's Sylvester matrix, per 128 x 128 tile),
    evaluated in float64 from the decoded values: planes on the right sides, both transforms, the scale.  bf16 rounding
    only (2^-8 relative), an all-zero plane gives (signed) zeros."""
    from scipy.linalg import hadamard
    rng = np.random.default_rng(42)
    rows, cols = 256, 384
    codes = rng.integers(0, 256, rows * cols // 2, dtype=np.uint8)
    suh = (rng.uniform(0.5, 1.5, cols) * rng.choice([-1, 1], cols)).astype(np.float16).astype(np.float32)
    svh = (rng.uniform(0.5, 1.5, rows) * rng.choice([-1, 1], rows)).astype(np.float16).astype(np.float32)
    G = oracle.ht_decode(codes, rows, cols).astype(np.float64)
    H = hadamard(128).astype(np.float64)
    W = np.empty((rows, cols))
    for r in range(0, rows, 128):
        for c in range(0, cols, 128):
            W[r:r + 128, c:c + 128] = H @ G[r:r + 128, c:c + 128] @ H / 128.0
    W = W * svh[:, None].astype(np.float64) * suh[None, :].astype(np.float64)
    got = _bf16_to_f64(oracle.v2_dense_bf16(16, codes, rows, cols, suh, svh))
    assert np.abs(got - W).max() <= 2.0 ** -8 * np.abs(W).max()
    assert (np.abs(got - W) <= 2.0 ** -8 * np.abs(W) + 1e-6).all()
    assert not (oracle.v2_dense_bf16(16, codes, rows, cols, suh * 0, svh) & 0x7fff).any()


def test_v2_dense_q6g64_closed_form(oracle):
    """q6g64 rows packed here element by element from the published layout (row stride align16(13 C / 16): C/2 bytes of
    low nibbles, even column in the low half; C/4 bytes of high bit pairs, column k in byte k/4 at bits 2 (k % 4); C/64
    x (f16 scale, f16 bias)).  Scale 1 / bias 0: the matrix is the codes themselves (0 .. 63, exact in bf16).  General
    scales: code * scale + bias in float64 within bf16 rounding."""
    rng = np.random.default_rng(43)
    R, Cc = 5, 192
    st = (13 * Cc // 16 + 15) & ~15
    code = rng.integers(0, 64, (R, Cc))
    code[0, :64] = np.arange(64)
    for unit in (True, False):
        sc = np.ones((R, Cc // 64), np.float16) if unit else rng.uniform(0.01, 0.05, (R, Cc // 64)).astype(np.float16)
        bi = np.zeros((R, Cc // 64), np.float16) if unit else rng.uniform(-1, 1, (R, Cc // 64)).astype(np.float16)
        blob = np.zeros((R, st), np.uint8)
        for r in range(R):
            for k in range(Cc):
                blob[r, k // 2] |= (int(code[r, k]) & 15) << (4 * (k % 2))
                blob[r, Cc // 2 + k // 4] |= (int(code[r, k]) >> 4) << (2 * (k % 4))
            for g in range(Cc // 64):
                blob[r, 3 * Cc // 4 + 4 * g: 3 * Cc // 4 + 4 * g + 2] = np.frombuffer(sc[r, g].tobytes(), np.uint8)
                blob[r, 3 * Cc // 4 + 4 * g + 2: 3 * Cc // 4 + 4 * g + 4] = np.frombuffer(bi[r, g].tobytes(), np.uint8)
        got = _bf16_to_f64(oracle.v2_dense_bf16(24, blob, R, Cc))
        want = code * np.repeat(sc.astype(np.float64), 64, axis=1) + np.repeat(bi.astype(np.float64), 64, axis=1)
        if unit:
            assert (got == want).all()
        else:
            assert (np.abs(got - want) <= 2.0 ** -8 * np.abs(want) + 1e-9).all()
