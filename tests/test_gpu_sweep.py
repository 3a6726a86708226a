"""Randomised whole-layer parity sweep against the oracle: formats, codebooks, shapes, expert counts, top-k, router
dtypes, bias / shared expert / zero rows, expert scales from twenty times below to thirty times above the usual one,
and sequences of calls of different sizes on one context.  Fixed seeds; every case names itself in the assertion.
(The shapes and value regimes here are the ones an open-ended version of this sweep found defects with: a router
launch reading an absent gate vector, f16 intermediates leaving the normal range on either side.)"""
import os
import sys

import numpy as np
import pytest

from gfx1151_engine_amd import synth as S
from helpers import HostLayer, max_abs_rel

pytestmark = pytest.mark.gpu


def gpu(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def draw_codebook(rng, fmt):
    kind = str(rng.choice(["zp8", "affine", "universal", "table"])) if fmt == "q4cp" else "zp8"
    if kind == "affine":
        a, b = rng.uniform(0.2, 2.0), rng.uniform(-12, 2)
        return kind, (a * np.arange(16) + b).astype(np.float32)
    if kind == "universal":
        return kind, S.UNIVERSAL_CODEBOOK
    if kind == "table":
        return kind, np.sort(rng.standard_normal(16)).astype(np.float32)
    return kind, None


def tolerance(fmt, T):
    return 2e-3 if T > 32 else (5e-4 if fmt == "q4k" else 2e-4)


def check(m, oracle, ol, x, fmt, k, desc):
    if os.environ.get("MOE_SWEEP_TRACE"):  # name the case before its GPU work (past pytest's capture)
        sys.__stderr__.write(desc + "\n")
        sys.__stderr__.flush()
    T = x.shape[0]
    yo, io, wo = oracle.moe_layer(ol, x)
    y = m.forward(0, gpu(x)).cpu().numpy()
    ids, ws = m.last_routing(T)
    ids, ws = ids.cpu().numpy()[:, :k], ws.cpu().numpy()[:, :k]
    assert np.isfinite(y).all(), desc
    assert (ids == io[:, :k]).all(), desc
    assert np.abs(ws - wo[:, :k]).max() <= 1e-6, desc
    err = max_abs_rel(y, yo) if np.abs(yo).max() > 0 else float(np.abs(y).max())
    assert err <= tolerance(fmt, T), (desc, err)


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_single_calls(oracle, seed):
    from gfx1151_engine_amd import capi
    for ci in range(40):
        rng = np.random.default_rng(seed * 1000 + ci)
        fmt = str(rng.choice(["q4cp", "q4cp", "q4cp", "q4k", "i4r"]))
        batch = bool(rng.integers(0, 2))
        if fmt == "i4r":
            d, mid = int(rng.choice([256, 512, 1024])), int(rng.choice([256, 512, 768]))
        elif batch:
            d, mid = int(rng.choice([256, 384, 512, 1024, 1536])), int(rng.choice([256, 384, 512, 768]))
        else:
            d, mid = int(rng.choice([256, 320, 512, 1024, 3072])), int(rng.choice([256, 384, 768, 160 if fmt == "q4cp" else 256]))
        if fmt == "q4k":
            d, mid = (d + 255) // 256 * 256, (mid + 255) // 256 * 256
        E = int(rng.choice([8, 16, 33, 64, 100, 128]))
        k = min(int(rng.choice([1, 2, 4, 8, 10])), E - 1)
        T = int(rng.integers(33, 400)) if batch else int(rng.integers(1, 33))
        while batch and T * d * mid * (k + 1) > 1.5e9 and T > 40:
            T //= 2
        rdt = str(rng.choice(["f32", "bf16"]))
        cbk, codebook = draw_codebook(rng, fmt)
        sstd = float(rng.choice([0.01, 0.05, 0.002, 0.0005, 0.3]))
        shared = bool(rng.integers(0, 4) != 0)
        bias = S.zipf_bias(rng, E, 1.1, 1.0) if rng.integers(0, 2) else None
        xs = float(rng.choice([1.0, 0.3, 3.0]))
        intdec = int(rng.integers(0, 4) != 0)
        desc = (f"seed {seed} case {ci}: {fmt} d={d} mid={mid} E={E} k={k} T={T} router={rdt} codebook={cbk} scale={sstd} "
                f"shared={shared} bias={bias is not None} x*{xs} int_decode={intdec}")
        hl = HostLayer(rng, d, mid, E, k, fmt=fmt, router_dtype=rdt, codebook=codebook, scale_std=sstd, shared=shared, bias=bias)
        x = rng.standard_normal((T, d), dtype=np.float32) * xs
        if rng.integers(0, 3) == 0:
            x[rng.integers(0, T)] = 0.0
        m, dev = hl.to_gpu(max_tokens=max(T, 32))
        m.set_option(capi.OPT_INT_DECODE, intdec)
        check(m, oracle, hl.oracle_layer(), x, fmt, k, desc)
        m.close()


@pytest.mark.parametrize("seed", [21, 22])
def test_sequences_of_calls_on_one_context(oracle, seed):
    from gfx1151_engine_amd import capi
    for ci in range(25):
        rng = np.random.default_rng(seed * 1000 + ci)
        fmt = str(rng.choice(["q4cp", "q4cp", "q4k", "q4k", "i4r"]))
        if fmt == "i4r":
            d, mid = int(rng.choice([256, 512, 1024])), int(rng.choice([256, 512, 768]))
        else:
            d, mid = int(rng.choice([256, 512, 1024, 1536])), int(rng.choice([256, 512, 768]))
        gg = (12, 12, 12)
        if fmt == "q4k":
            d, mid = (d + 255) // 256 * 256, (mid + 255) // 256 * 256
            gg = [(12, 12, 12), (13, 8, 12), (12, 7, 12), (13, 7, 8), (12, 8, 13), (23, 20, 12), (13, 8, 13)][int(rng.integers(0, 7))]
        E = int(rng.choice([8, 16, 33, 64, 100]))
        k = min(int(rng.choice([1, 2, 4, 8, 10])), E - 1)
        rdt = str(rng.choice(["f32", "bf16"]))
        cbk, codebook = draw_codebook(rng, fmt)
        sstd = float(rng.choice([0.01, 0.05, 0.002]))
        shared = bool(rng.integers(0, 4) != 0)
        sdense = str(rng.choice(["bf16", "f32", "q8g64"])) if shared and rng.integers(0, 4) == 0 else None
        bias = S.zipf_bias(rng, E, 1.1, 1.0) if rng.integers(0, 2) else None
        Tmax = int(rng.choice([32, 40, 64, 200, 333]))
        while Tmax * d * mid * (k + 1) > 1.2e9 and Tmax > 40:
            Tmax //= 2
        seq = []
        for _ in range(int(rng.integers(3, 6))):
            c = int(rng.integers(0, 6))
            T = [1, Tmax, int(rng.integers(1, 33)), min(Tmax, 33), int(rng.integers(1, Tmax + 1)),
                 min(Tmax, int(rng.choice([4, 5, 24, 25, 32])))][c]
            seq.append((T, int(rng.integers(0, 4) != 0)))
        hl = HostLayer(rng, d, mid, E, k, fmt=fmt, router_dtype=rdt, codebook=codebook, scale_std=sstd, shared=shared,
                       bias=bias, gg_types=gg, shared_dense=sdense)
        ol = hl.oracle_layer()
        m, dev = hl.to_gpu(max_tokens=Tmax)
        for T, intdec in seq:
            desc = (f"seed {seed} case {ci}: {fmt} types={gg} d={d} mid={mid} E={E} k={k} router={rdt} codebook={cbk} "
                    f"scale={sstd} shared={shared} dense={sdense} bias={bias is not None} max_tokens={Tmax} calls={seq} at T={T}")
            m.set_option(capi.OPT_INT_DECODE, intdec)
            check(m, oracle, ol, rng.standard_normal((T, d), dtype=np.float32), fmt, k, desc)
        m.close()
