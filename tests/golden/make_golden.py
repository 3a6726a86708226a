"""Writes tests/golden/*.npz from the reference's OWN code (oracle/_ref/libmoe_ref.so, built by
oracle/Makefile from the reference tree where it lies).  Run in the build container only:

    python tests/golden/make_golden.py

Every fixture is data: seeded inputs in the engine's byte layouts plus the outputs the reference's
functions produced for them (hgn::Checkpoint::q4cp_row, gguf::dequant_row / scale_min_k4,
hgn::fp16_to_f32, and Model::moe of src/ref.cpp on a one-layer synthetic checkpoint).
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from gfx1151_engine_amd import synth as S  # noqa: E402
from oracle import oracle as O  # noqa: E402

OUT = os.path.dirname(os.path.abspath(__file__))


def fp16_table():
    h = np.arange(65536, dtype=np.uint32)
    r = O.ref()
    v = np.array([r.ref_fp16_to_f32(int(x)) for x in h], dtype=np.float32)
    np.savez_compressed(os.path.join(OUT, "fp16_table.npz"), bits=v.view(np.uint32))


def q4cp_cases():
    rng = np.random.default_rng(20250101)
    out = {}
    # (rows, cols): 640 exercises the padded scale record (40 B -> 48 B), 96 a short one
    for i, (rows, cols) in enumerate([(6, 640), (5, 96), (4, 3072), (8, 768)]):
        cb = rng.uniform(-2, 2, 16).astype(np.float32) if i % 2 == 0 else S.ZP8_CODEBOOK
        scales = (np.abs(rng.standard_normal((rows, cols // 32))) * 0.01).astype(np.float16)
        # special scales: zero, negative zero, smallest subnormal, largest subnormal, max normal, negative
        sp = np.array([0x0000, 0x8000, 0x0001, 0x03ff, 0x7bff, 0xb555], np.uint16).view(np.float16)
        scales.reshape(-1)[:sp.size] = sp
        blob = S.make_q4cp(rng, rows, cols, codebook=cb, scales=scales)
        # make sure all 16 codes occur next to every special scale
        blob[64:64 + 16] = np.arange(16, dtype=np.uint8) * 17
        out[f"blob{i}"] = blob
        out[f"shape{i}"] = np.array([rows, cols])
        out[f"bits{i}"] = O.ref_q4cp_rows(blob, rows, cols, 0, rows).view(np.uint32)
    out["n"] = np.array(4)
    np.savez_compressed(os.path.join(OUT, "q4cp_rows.npz"), **out)


def q4k_cases():
    rng = np.random.default_rng(20250102)
    out = {}
    for i, (rows, cols) in enumerate([(3, 256), (2, 768), (2, 3072)]):
        raw = S.make_q4k(rng, rows, cols)
        out[f"raw{i}"] = raw
        out[f"shape{i}"] = np.array([rows, cols])
        out[f"bits{i}"] = O.ref_q4k_rows(raw, rows, cols).view(np.uint32)
    out["n"] = np.array(3)
    # scale_min_k4 on random 12-byte records, all 8 sub-blocks
    q = rng.integers(0, 256, (64, 12), dtype=np.uint8)
    sm = np.array([[O.ref_scale_min_k4(j, q[i]) for j in range(8)] for i in range(64)], np.uint8)
    out["k4_q"] = q
    out["k4_sm"] = sm
    np.savez_compressed(os.path.join(OUT, "q4k_rows.npz"), **out)


def layer_cases():
    """Model::moe on tiny layers: (d, mid, E, k, router/shared dtype)."""
    out = {}
    cases = [(64, 32, 8, 3, "bf16"), (128, 64, 8, 4, "q4cp"), (96, 64, 12, 10, "bf16"),
             (128, 64, 8, 3, "q8g64")]
    for i, (d, mid, E, k, kind) in enumerate(cases):
        rng = np.random.default_rng(777 + i)
        cb = rng.uniform(-2, 2, 16).astype(np.float32) if i == 2 else None
        gu = S.make_q4cp(rng, E * 2 * mid, d, codebook=cb, scale_std=0.05)
        dn = S.make_q4cp(rng, E * d, mid, codebook=cb, scale_std=0.05)
        router = S.f32_to_bf16_bits(rng.standard_normal((E, d)).astype(np.float32) * 0.2)
        sg = S.f32_to_bf16_bits(rng.standard_normal((1, d)).astype(np.float32) * 0.2)
        if kind == "q4cp":
            shg, shu, shd = (S.make_q4cp(rng, mid, d, scale_std=0.05), S.make_q4cp(rng, mid, d, scale_std=0.05),
                             S.make_q4cp(rng, d, mid, scale_std=0.05))
            sh_dt = O.Q4CP
        elif kind == "q8g64":  # the overlay files' storage of the shared expert (src/hgn.h:10, src/ref.cpp:91-106)
            shg, shu, shd = (S.make_q8g64(rng, mid, d, 0.1), S.make_q8g64(rng, mid, d, 0.1), S.make_q8g64(rng, d, mid, 0.1))
            sh_dt = O.Q8G64
        else:
            shg = S.f32_to_bf16_bits(rng.standard_normal((mid, d)).astype(np.float32) * 0.1)
            shu = S.f32_to_bf16_bits(rng.standard_normal((mid, d)).astype(np.float32) * 0.1)
            shd = S.f32_to_bf16_bits(rng.standard_normal((d, mid)).astype(np.float32) * 0.1)
            sh_dt = O.BF16
        layer = O.Layer(d, mid, E, k, O.Mat(O.BF16, router, E, d), O.Mat(O.Q4CP, dn, E * d, mid),
                        gate_up=O.Mat(O.Q4CP, gu, E * 2 * mid, d),
                        shared=[O.Mat(sh_dt, shg, mid, d), O.Mat(sh_dt, shu, mid, d), O.Mat(sh_dt, shd, d, mid),
                                O.Mat(O.BF16, sg, 1, d)])
        T = 6
        x = rng.standard_normal((T, d)).astype(np.float32)
        if i == 0:
            x[5] = 0.0  # all-zero token: uniform router probabilities -> ties -> lowest indices
        y = np.stack([O.ref_moe_token(layer, x[t]) for t in range(T)])
        out.update({f"cfg{i}": np.array([d, mid, E, k, sh_dt]), f"gu{i}": gu, f"dn{i}": dn, f"router{i}": router,
                    f"sg{i}": sg, f"shg{i}": np.asarray(shg), f"shu{i}": np.asarray(shu), f"shd{i}": np.asarray(shd),
                    f"x{i}": x, f"ybits{i}": y.view(np.uint32)})
    out["n"] = np.array(len(cases))
    # Checkpoint::dequant of one q8g64 tensor (src/hgn.h:189-202)
    rng = np.random.default_rng(790)
    q8 = S.make_q8g64(rng, 5, 192, 0.3)
    out["q8g64_raw"] = q8
    out["q8g64_bits"] = O.ref_dequant_tensor(O.Mat(O.Q8G64, q8, 5, 192)).view(np.uint32)
    # Checkpoint::dequant of one planar q8g32 tensor (src/hgn.h:176-183)
    q8p = S.quantize_q8g32(rng.standard_normal((6, 96)).astype(np.float32) * 0.3)
    out["q8g32_raw"] = q8p
    out["q8g32_bits"] = O.ref_dequant_tensor(O.Mat(O.Q8G32, q8p, 6, 96)).view(np.uint32)
    np.savez_compressed(os.path.join(OUT, "moe_layer.npz"), **out)


if __name__ == "__main__":
    assert O.ref() is not None, "oracle/_ref/libmoe_ref.so missing: run `make -C oracle`"
    fp16_table()
    q4cp_cases()
    q4k_cases()
    layer_cases()
    for f in sorted(os.listdir(OUT)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(OUT, f)))
