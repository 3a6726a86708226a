"""GPU parity of the whole layer through moe_forward against the oracle (the restated
src/ref.cpp Model::moe): router ids bit-exact, y within max-abs-rel 2e-3 (the small-batch f32
kernels are held to 1e-4, the integer-dot kernels to 2e-4 (q4cp) and 5e-4 (Q4_K))."""
import zlib

import numpy as np
import pytest

from gfx1151_engine_amd import synth as S

from helpers import HostLayer, bits, max_abs_rel

pytestmark = pytest.mark.gpu

TOL_LAYER = 2e-3   # stated tolerance for the layer (f16/bf16 MFMA path)
TOL_GEMV = 1e-4    # small-batch GEMV path, f32 kernels
TOL_INT_Q4CP = 2e-4  # integer-dot kernels, q4cp: activations as four 4-bit digit planes per 32-group (worst of
                     # 60 seeds at one token: 7.8e-5)
TOL_INT_Q4K = 5e-4  # integer-dot kernels on raw Q4_K blocks: activations as two 8-bit digit planes per
                    # 32-group; the unsigned codes (w = d*sc*n - dmin*m, n in 0..15) double the weight of
                    # the activations' rounding against the zero-centred q4cp codes (worst of 80 seeds: 2.4e-4)


def tol_small(fmt):
    return TOL_INT_Q4K if fmt == "q4k" else TOL_INT_Q4CP


def gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_layer(hl, x, max_tokens=None):
    m, dev = hl.to_gpu(max_tokens=max_tokens or max(32, x.shape[0]))
    y = m.forward(0, gpu(x))
    ids, ws = m.last_routing(x.shape[0])
    out = y.cpu().numpy(), ids.cpu().numpy(), ws.cpu().numpy()
    m.close()
    return out


@pytest.mark.parametrize("fmt,d,mid,E,k,T,cb", [
    ("q4cp", 3072, 768, 32, 10, 1, None), ("q4cp", 3072, 768, 32, 10, 20, None),
    ("q4cp", 640, 160, 16, 4, 7, "random"), ("q4k", 3072, 768, 24, 10, 1, None),
    ("q4k", 3072, 768, 24, 10, 20, None), ("q4k", 256, 256, 8, 3, 5, None)])
def test_small_batch_layer(oracle, fmt, d, mid, E, k, T, cb):
    rng = np.random.default_rng(zlib.crc32(f"{fmt}-{d}-{T}".encode()))  # (hash() of a str changes per process)
    codebook = rng.uniform(-2, 2, 16).astype(np.float32) if cb == "random" else None
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt, codebook=codebook)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    y, ids, ws = run_layer(hl, x)
    assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 1e-6
    assert max_abs_rel(y, yo) <= tol_small(fmt), max_abs_rel(y, yo)


TOL_LUT = 2e-5  # look-up kernels for codebooks that are not a*n + b: f32 throughout (f32 sums against the
                # reference's fp64 ones; the order of the additions is the only difference from the f32 GEMV kernels)


@pytest.mark.parametrize("T", [1, 2, 5, 6, 20, 32])
@pytest.mark.parametrize("kind", ["universal", "random"])
def test_small_batch_table_codebooks(oracle, T, kind):
    """The reference converter's fixed non-uniform table (tools/flashnext2hgn.py:530-531) in every routed-expert
    tensor, and a table of its own in each of the shared expert's tensors (:164-187): the look-up decode kernels
    against the oracle, and the plain f32 kernels (MOE_OPT_INT_DECODE = 0) as a second opinion."""
    import torch
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(500 + T)
    d, mid, E, k = 3072, 768, 24, 10
    cb = S.UNIVERSAL_CODEBOOK if kind == "universal" else np.sort(rng.standard_normal(16)).astype(np.float32)
    scb = [np.sort(rng.standard_normal(16)).astype(np.float32) * (0.5 + i) for i in range(3)]
    hl = HostLayer(rng, d, mid, E, k, codebook=cb, shared_codebooks=scb, scale_std=0.05)
    x = rng.standard_normal((T, d), dtype=np.float32)
    x[0] *= 300.0  # (each 32-group of activations is rescaled by a power of two on its way to f16)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=32)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, ws = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    assert np.abs(ws.cpu().numpy()[:, :k] - wo[:, :k]).max() <= 1e-6
    err = max(max_abs_rel(y[t], yo[t]) for t in range(T))  # per token: token 0 is 300 times larger
    assert err <= TOL_LUT, err  # (up to 5 tokens the look-up kernels, beyond that the plain f32 kernels)
    m.set_option(capi.OPT_INT_DECODE, 0)
    y2 = m.forward(0, gpu(x)).cpu().numpy()
    assert max(max_abs_rel(y2[t], yo[t]) for t in range(T)) <= TOL_GEMV
    m.close()


@pytest.mark.parametrize("limit", [0, 3, 32])
@pytest.mark.parametrize("codebook", ["affine", "universal"])
def test_f32_decode_token_limit(oracle, limit, codebook):
    """MOE_OPT_F32_DECODE_MAX_TOKENS moves the batch size at which the f32 path's down launch changes from the
    register-resident kernel to the plain one: every setting gives the oracle's ids and meets the f32 bar at 2, 4 and
    20 tokens (affine codebook with the integer-dot kernels off; the converter's table with them on)."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(9100 + limit)
    d, mid, E, k = 3072, 768, 24, 10
    hl = HostLayer(rng, d, mid, E, k, codebook=S.UNIVERSAL_CODEBOOK, scale_std=0.05) if codebook == "universal" else \
        HostLayer(rng, d, mid, E, k)
    m, dev = hl.to_gpu(max_tokens=32)
    if codebook == "affine":
        m.set_option(capi.OPT_INT_DECODE, 0)
    m.set_option(capi.OPT_F32_DECODE_MAX_TOKENS, limit)
    for T in (2, 4, 20):
        x = rng.standard_normal((T, d), dtype=np.float32)
        yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
        y = m.forward(0, gpu(x)).cpu().numpy()
        ids, ws = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all(), T
        assert np.abs(ws.cpu().numpy()[:, :k] - wo[:, :k]).max() <= 1e-6
        assert max_abs_rel(y, yo) <= TOL_GEMV, (T, max_abs_rel(y, yo))
    with pytest.raises(capi.MoeError):
        m.set_option(capi.OPT_F32_DECODE_MAX_TOKENS, 33)
    m.close()


@pytest.mark.parametrize("fmt,T,rdt", [("q4cp", 3, "f32"), ("q4cp", 32, "f32"), ("q4k", 27, "f32"), ("q4k", 2, "f32"),
                                        ("q4cp", 1, "bf16"), ("q4cp", 4, "bf16"), ("q4cp", 5, "f32"), ("q4cp", 11, "f32"), ("q4cp", 12, "bf16"), ("q4cp", 17, "f32"),
                                        ("q4k", 30, "bf16")])
def test_small_batch_sizes_and_router_dtypes(oracle, fmt, T, rdt):
    """The token counts at which the small path changes kernels (1 / 2-4 / 5-24 / 25-32: the logits
    launch differs, above 24 tokens it is split in two) with f32 and bf16 router matrices."""
    rng = np.random.default_rng(4242 + 7 * T + (rdt == "bf16"))
    d, mid, E, k = 3072, 768, 24, 10
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt, router_dtype=rdt)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    y, ids, ws = run_layer(hl, x)
    assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 1e-6
    assert max_abs_rel(y, yo) <= tol_small(fmt), max_abs_rel(y, yo)


@pytest.mark.parametrize("T", [3, 6, 12, 21, 30])
@pytest.mark.parametrize("rdt", ["f32", "bf16"])
def test_small_batch_router_without_gate_vector_and_ragged_rows(oracle, T, rdt):
    """A layer without a shared expert (no gate vector beside the router matrix) whose expert count is not a multiple
    of the router launch's rows per block, at a width where 5..24 tokens take the row-per-wave launch (d not a
    multiple of 256): the padding rows of the last block read the router matrix, never the absent gate vector."""
    rng = np.random.default_rng(3300 + T + (rdt == "bf16"))
    d, mid, E, k = 320, 256, 33, 4
    hl = HostLayer(rng, d, mid, E, k, router_dtype=rdt, shared=False,
                   bias=rng.standard_normal(E).astype(np.float32) * 0.1)
    x = rng.standard_normal((T, d), dtype=np.float32) * 3
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    y, ids, ws = run_layer(hl, x)
    assert (ids[:, :k] == io[:, :k]).all(), "router ids must be bit-exact"
    assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 1e-6
    assert max_abs_rel(y, yo) <= TOL_INT_Q4CP, max_abs_rel(y, yo)


@pytest.mark.parametrize("fmt,T", [("q4cp", 1), ("q4cp", 3), ("q4cp", 5), ("q4cp", 6), ("q4cp", 9), ("q4cp", 32),
                                   ("q4k", 1), ("q4k", 9)])
def test_int_decode_switch(oracle, fmt, T):
    """MOE_OPT_INT_DECODE 1 (integer-dot kernels, default) and 0 (f32 kernels) both meet the GEMV bar
    and select the same experts.  (q4cp with the switch at 0: up to 4 tokens the register-resident f32 kernels with
    the top-k inside the gate/up launch, at 5 with the ids from the router's launches, from 6 on the plain f32 down
    kernel behind the register-resident gate/up launch.)"""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(77 + T)
    d, mid, E, k = 3072, 768, 16, 10
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt)
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=32)
    ys = []
    for opt in (1, 0):
        m.set_option(capi.OPT_INT_DECODE, opt)
        y = m.forward(0, gpu(x)).cpu().numpy()
        ids, _ = m.last_routing(T)
        assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
        assert max_abs_rel(y, yo) <= (tol_small(fmt) if opt else TOL_GEMV), (opt, max_abs_rel(y, yo))
        ys.append(y)
    assert not (ys[0] == ys[1]).all(), "the two paths are different kernels (digit planes vs f32)"
    m.close()


@pytest.mark.parametrize("fmt,T", [("q4cp", 1), ("q4cp", 6), ("q4k", 1), ("q4k", 3)])
def test_decode_topk_near_ties(oracle, fmt, T):
    """The decode gate/up kernels rank the experts by logit and fall back to the exact softmax selection when two
    of the k + 1 best logits are closer than 1e-6.  Router rows repeated (equal logits: the lower index must come
    first, and a copy may sit on the rank k / k + 1 boundary) and rows that differ in the last bits force that
    fallback; ids and order must still be the oracle's."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(17 + T)
    d, mid, E, k = (3072, 768, 24, 10) if fmt == "q4cp" else (512, 256, 24, 10)
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt)
    hl.router[7] = hl.router[3]
    hl.router[20] = hl.router[3]
    hl.router[11] = hl.router[5]
    hl.router[16] = hl.router[5] * np.float32(1 + 2 ** -22)
    hl.router[2] = hl.router[9]
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=8)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, ws = m.last_routing(T)
    ids, ws = ids.cpu().numpy(), ws.cpu().numpy()
    assert (ids[:, :k] == io[:, :k]).all(), (ids[:, :k], io[:, :k])
    assert np.abs(ws[:, :k] - wo[:, :k]).max() <= 1e-6
    assert max_abs_rel(y, yo) <= tol_small(fmt), max_abs_rel(y, yo)
    m.close()


@pytest.mark.parametrize("fmt", ["q4cp", "q4k"])
def test_decode_topk_wide_logit_range(oracle, fmt):
    """Router rows scaled so that the logits span hundreds: below the best few, the reference's f32 probabilities
    go subnormal or to zero and tie, and ties are ordered by expert index.  The gate/up launch of the decode path
    (which ranks by logit) and the down launch (which takes the ids of the exact selection) must still agree with
    each other and with the oracle: a slot that ran gate/up for one expert and down for another shows in y."""
    rng = np.random.default_rng(29)
    d, mid, E, k = (3072, 768, 24, 10) if fmt == "q4cp" else (512, 256, 24, 10)
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt)
    # rows in descending-logit order that runs AGAINST the index order: ties between underflowed probabilities
    # then come out by index, i.e. opposite to the logits
    x = rng.standard_normal((3, d), dtype=np.float32)
    u = x[0] / np.linalg.norm(x[0])
    hl.router[:] = 1e-3 * rng.standard_normal((E, d), dtype=np.float32)
    hl.router += np.outer(np.linspace(-9.0, 3.0, E), u).astype(np.float32)  # token 0: logits ~ 55 * (-9 .. 3)
    x[2] = 0.0                                                                # token 2: all logits equal
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    lg = oracle.router(hl.oracle_layer().router, x, k)[0]
    assert lg[0].max() - np.sort(lg[0])[-k] > 90, "the k-th logit of token 0 must lie in the underflow range"
    m, dev = hl.to_gpu(max_tokens=8)
    for T in (1, 3):
        y = m.forward(0, gpu(x[:T])).cpu().numpy()
        ids, ws = m.last_routing(T)
        ids, ws = ids.cpu().numpy(), ws.cpu().numpy()
        assert (ids[:, :k] == io[:T, :k]).all(), (T, ids[:, :k], io[:T, :k])
        assert np.abs(ws[:, :k] - wo[:T, :k]).max() <= 1e-6
        assert max_abs_rel(y, yo[:T]) <= tol_small(fmt), (T, max_abs_rel(y, yo[:T]))
    m.close()


@pytest.mark.parametrize("tgu,tdn,tsh,T", [(13, 8, 12, 1), (12, 7, 12, 5), (13, 7, 8, 3), (12, 8, 13, 40), (23, 20, 12, 2),
                                            (20, 23, 23, 7), (13, 8, 8, 1), (13, 8, 8, 20), (12, 7, 7, 32), (8, 13, 7, 2),
                                            (20, 20, 20, 1), (23, 23, 23, 4), (23, 20, 8, 19), (12, 23, 20, 30)])
def test_gguf_mixed_types(oracle, tgu, tdn, tsh, T):
    """GGUF layers in the type mix of the reference's checkpoints (Q4_K / Q5_K gate and up, Q5_1 / Q8_0 down, a Q8_0
    shared expert; src/gpu/parts/30_host_util.inc:399-405, src/gguf_map.h:212-214) and in the IQ4_NL / IQ4_XS types
    (src/gguf.h:376-407): every mix takes the integer-dot decode kernels (and, with MOE_OPT_INT_DECODE = 0, the general
    f32 GEMV kernels); ids bit-exact; T = 40 is a batch for the general grouped GEMM."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(tgu * 100 + tdn * 10 + T)
    d, mid, E, k = 512, 256, 12, 4
    hl = HostLayer(rng, d, mid, E, k, fmt="q4k", gg_types=(tgu, tdn, tsh))
    x = rng.standard_normal((T, d), dtype=np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=64)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, ws = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    assert np.abs(ws.cpu().numpy()[:, :k] - wo[:, :k]).max() <= 1e-6
    # batches over 32 tokens take the general grouped GEMM (f16 MFMA operands): the batch tolerance
    tol = 2e-3 if T > 32 else TOL_INT_Q4K
    assert max_abs_rel(y, yo) <= tol, max_abs_rel(y, yo)
    if T <= 32:
        m.set_option(capi.OPT_INT_DECODE, 0)
        y2 = m.forward(0, gpu(x)).cpu().numpy()
        assert max_abs_rel(y2, yo) <= TOL_GEMV, max_abs_rel(y2, yo)
    m.close()


@pytest.mark.parametrize("share", [0.3, 1.0])
def test_unique_expert_path(oracle, share):
    """MOE_OPT_UNIQUE_MIN_TOKENS: a verify-size batch through the expert-sorted pair lists (every distinct
    expert read once) gives the same experts and, within the GEMV bar, the same output."""
    import torch
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(91)
    d, mid, E, k, T = 3072, 768, 24, 10, 20
    hl = HostLayer(rng, d, mid, E, k)
    x = rng.standard_normal((T, d), dtype=np.float32)
    n = int(round(share * T))
    for i in range(1, n):  # drafted tokens that reproduce the template token's routing
        x[i] = x[0] + 1e-3 * rng.standard_normal(d).astype(np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=32)
    m.set_option(capi.OPT_UNIQUE_MIN_TOKENS, 8)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, _ = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    assert max_abs_rel(y, yo) <= TOL_INT_Q4CP, max_abs_rel(y, yo)
    m.set_option(capi.OPT_UNIQUE_MIN_TOKENS, 0)
    y2 = m.forward(0, gpu(x)).cpu().numpy()
    assert max_abs_rel(y2, yo) <= TOL_INT_Q4CP
    m.close()


@pytest.mark.parametrize("types,T,share,shared", [((12, 12, 12), 20, 0.3, True), ((13, 8, 8), 20, 1.0, True),
                                                  ((12, 7, 13), 12, 0.3, True), ((13, 8, 8), 32, 0.5, False),
                                                  ((8, 13, 7), 17, 0.0, True)])
def test_unique_expert_path_gguf(oracle, types, T, share, shared):
    """The distinct-expert kernels for GGUF layers (any mix of Q4_K / Q5_K / Q8_0 / Q5_1): a verify-size batch through
    the expert-sorted pair lists, tiles of at most four pairs, against the oracle and against the per-token kernels."""
    import torch
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(92 + T)
    d, mid, E, k = 3072, 768, 24, 10
    hl = HostLayer(rng, d, mid, E, k, fmt="q4k", gg_types=types, shared=shared)
    x = rng.standard_normal((T, d), dtype=np.float32)
    for i in range(1, int(round(share * T))):
        x[i] = x[0] + 1e-3 * rng.standard_normal(d).astype(np.float32)
    yo, io, wo = oracle.moe_layer(hl.oracle_layer(), x)
    m, dev = hl.to_gpu(max_tokens=32)
    m.set_option(capi.OPT_UNIQUE_MIN_TOKENS, 8)
    m.set_option(capi.OPT_UNIQUE_GGUF, 1)
    m.profile(True)
    y = m.forward(0, gpu(x)).cpu().numpy()
    assert m.profile_read()["reduce"] > 0, "the distinct-expert path ends in a combine launch"
    m.profile(False)
    ids, ws = m.last_routing(T)
    assert (ids.cpu().numpy()[:, :k] == io[:, :k]).all()
    assert np.abs(ws.cpu().numpy()[:, :k] - wo[:, :k]).max() <= 1e-6
    assert max_abs_rel(y, yo) <= TOL_INT_Q4K, max_abs_rel(y, yo)
    m.set_option(capi.OPT_UNIQUE_GGUF, 0)
    y2 = m.forward(0, gpu(x)).cpu().numpy()
    assert max_abs_rel(y2, yo) <= TOL_INT_Q4K
    assert max_abs_rel(y, y2) <= 1e-5, "the same integer sums per pair: only the order of the combine's additions differs"
    m.close()


@pytest.mark.parametrize("i", [0, 1, 2, 3])
def test_golden_layers_from_reference(oracle, golden, i):
    """Inputs and outputs of the reference's own Model::moe (tests/golden/moe_layer.npz): four layers, two of them
    with a bf16 shared expert, one with a q8g64 one."""
    import torch
    from gfx1151_engine_amd import capi
    g = golden("moe_layer.npz")
    assert int(g["n"]) == 4
    d, mid, E, k, sh_dt = (int(v) for v in g[f"cfg{i}"])
    m = capi.Moe(d, mid, E, k)
    sh16 = sh_dt == oracle.BF16  # bf16 matrices are stored as uint16 bit patterns
    shv = [g[f"shg{i}"], g[f"shu{i}"], g[f"shd{i}"]]
    keep = [gpu(g[f"router{i}"].view(np.int16)), gpu(g[f"gu{i}"]), gpu(g[f"dn{i}"])] + \
           [gpu(a.view(np.int16) if sh16 else a) for a in shv] + [gpu(g[f"sg{i}"].view(np.int16))]
    wt = {oracle.BF16: capi.BF16, oracle.Q4CP: capi.Q4CP, oracle.Q8G64: capi.Q8G64}[sh_dt]
    m.set_router(0, capi.wview(keep[0], capi.BF16, E, d))
    m.set_experts_q4cp(0, capi.wview(keep[1], capi.Q4CP, E * 2 * mid, d), capi.wview(keep[2], capi.Q4CP, E * d, mid))
    m.set_shared(0, capi.wview(keep[3], wt, mid, d), capi.wview(keep[4], wt, mid, d),
                 capi.wview(keep[5], wt, d, mid), capi.wview(keep[6], capi.BF16, 1, d))
    x = g[f"x{i}"]
    want = g[f"ybits{i}"].view(np.float32)
    y = m.forward(0, gpu(x)).cpu().numpy()
    assert max_abs_rel(y, want) <= TOL_INT_Q4CP, i  # integer-dot decode kernels where the codebook is affine
    m.set_option(capi.OPT_INT_DECODE, 0)
    y = m.forward(0, gpu(x)).cpu().numpy()
    assert max_abs_rel(y, want) <= 5e-6, i          # f32 kernels: f32 against the reference's fp64 sums
    m.close()


def test_forward_errors(oracle):
    import torch
    from gfx1151_engine_amd import capi
    m = capi.Moe(256, 64, 8, 2, max_tokens=4)
    x = torch.zeros((2, 256), device="cuda")
    with pytest.raises(capi.MoeError):  # no weights registered
        m.forward(0, x)
    with pytest.raises(capi.MoeError):  # bad layer index
        m.forward(3, x)
    m.close()
    with pytest.raises(capi.MoeError):  # d not a multiple of 32
        capi.Moe(100, 64, 8, 2)


def test_stage_skipping_is_not_in_the_default_build_and_guarded_in_the_timing_twin():
    """MOE_OPT_TIMING_SKIP_STAGE makes a call return wrong results: the default library refuses it outright; the
    benchmark's timing twin takes it only once a complete call of that size has filled the scratch that the stages
    behind the skipped one index with."""
    import os
    import torch
    from gfx1151_engine_amd import LIB_TIMING, capi
    rng = np.random.default_rng(11)
    hl = HostLayer(rng, 1024, 256, 16, 4)
    m, dev = hl.to_gpu(max_tokens=8)
    with pytest.raises(capi.MoeError, match="unsupported"):
        m.set_option(capi.OPT_TIMING_SKIP_STAGE, 3)
    m.close()
    if not os.path.exists(LIB_TIMING):
        pytest.skip("timing twin of the library not built")
    twin = capi.second_binding(LIB_TIMING)
    mt, dev2 = hl.to_gpu(max_tokens=8, binding=twin)
    with pytest.raises(twin.MoeError, match="not ready"):
        mt.set_option(capi.OPT_TIMING_SKIP_STAGE, 3)  # fresh context: nothing has run yet
    x1 = torch.from_numpy(rng.standard_normal((1, 1024), dtype=np.float32)).cuda()
    x2 = torch.from_numpy(rng.standard_normal((2, 1024), dtype=np.float32)).cuda()
    y_full = mt.forward(0, x1).clone()
    mt.set_option(capi.OPT_TIMING_SKIP_STAGE, 3)
    mt.forward(0, x1)                       # runs (on the scratch of the complete call)
    with pytest.raises(twin.MoeError, match="not ready"):
        mt.forward(0, x2)                   # no complete call of two tokens yet
    mt.set_option(capi.OPT_TIMING_SKIP_STAGE, 0)
    assert torch.equal(mt.forward(0, x1), y_full)
    torch.cuda.synchronize()
    mt.close()


@pytest.mark.parametrize("fmt,T,int_decode", [("q4cp", 1, 1), ("q4cp", 3, 1), ("q4cp", 7, 1), ("q4cp", 20, 1),
                                               ("q4cp", 2, 0), ("q4k", 1, 1), ("q4k", 6, 1)])
def test_small_batch_ids_when_summation_orders_disagree(oracle, fmt, T, int_decode):
    """The small-batch router sums a logit's products lane-parallel, the reference one after the other
    (src/ref.cpp:70-77); the two fp64 sums can differ, and with them the f32 logits.  Here they differ by far more
    than an ulp: token activations with +-2^36 in two columns that cancel in one expert's row, so that the order of
    the additions decides what is left of the small terms.  A ladder of experts whose logits are pure biases, 1e-5
    apart, brackets that expert's sequential logit; wherever the parallel sum lands, its rank in the ladder is not
    the reference's.  The library must notice that the gaps are within what the two orders can differ by (a bound
    from the norms of the operands), recompute the logits in the reference's order and return the oracle's ids."""
    from gfx1151_engine_amd import capi
    rng = np.random.default_rng(101 + T)
    d, mid, E, k = 1024, 256, 64, 8
    bias = np.full(E, -30.0, np.float32)
    hl = HostLayer(rng, d, mid, E, k, fmt=fmt, bias=bias)
    A = 61                                     # the expert with the ill-conditioned sum (a high index: ties go to lower ones)
    hl.router[:] = 0.0
    hl.router[A] = rng.standard_normal(d).astype(np.float32) * np.float32(0.05)
    hl.router[A, 0] = 1.0
    hl.router[A, d - 1] = 1.0
    x = rng.standard_normal((T, d), dtype=np.float32)
    x[:, 0] = np.float32(2.0 ** 36)
    x[:, d - 1] = -np.float32(2.0 ** 36)
    bias[A] = 0.0
    # the sequential logit of A for token 0, then the ladder around it (every token sees the same ladder; the
    # tokens' own values of A differ, so A's rank differs from token to token)
    lgA = oracle.router(hl.oracle_layer().router, x, k, bias=bias)[0][:, A]
    ladder = [e for e in range(E) if e != A][:40]
    for j, e in enumerate(ladder):
        bias[e] = np.float32(np.float64(lgA[0]) + (3.5 - j) * 1e-5)  # four rungs above A's logit, the others below
    hl.bias = bias
    ol = hl.oracle_layer()
    lg, io, wo = oracle.router(ol.router, x, k, bias=bias)
    # the parallel-order logits of the stateless entry point (the forward call's launches use other splits of the
    # sum, with other roundings): they must not agree with the sequential ones, or the test tests nothing
    import torch
    Wd = torch.from_numpy(hl.router).cuda()
    lt = capi.router_logits(capi.wview(Wd, capi.F32, E, d), torch.from_numpy(x).cuda(), torch.from_numpy(bias).cuda(), mode=0).cpu().numpy()
    assert np.abs(lt[:, A].astype(np.float64) - lg[:, A]).max() > 2e-5, "the two summation orders (nearly) agree on this input: nothing to test"
    m, dev = hl.to_gpu(max_tokens=32)
    m.set_option(capi.OPT_INT_DECODE, int_decode)
    y = m.forward(0, torch.from_numpy(x).cuda())
    ids, ws = m.last_routing(T)
    torch.cuda.synchronize()
    ids = ids.cpu().numpy()
    assert (ids[:, :k] == io[:, :k]).all(), (ids[:, :k], io[:, :k])
    assert np.isfinite(y.cpu().numpy()).all()
    m.close()
