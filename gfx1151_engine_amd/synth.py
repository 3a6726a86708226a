"""Seeded synthetic tensors in the engine's on-disk byte layouts (numpy, host side).

q4cp blob  (hgn dtype 5, reference src/hgn.h:2-9,219-240):
    [64 B: 16 x f32 codebook][rows*cols/2 B codes, row-major, low nibble first]
    [rows x scale_stride B: cols/32 fp16 scales, record padded to 16 B]
Q4_K rows  (GGUF type 12, reference src/gguf.h:408-441): cols/256 super-blocks of 144 B:
    [fp16 d][fp16 dmin][12 B packed 6-bit scales/mins][128 B codes]
"""
import numpy as np

ZP8_CODEBOOK = np.arange(16, dtype=np.float32) - 8.0  # zero-point 8: w = (code - 8) * scale


def q4cp_scale_stride(cols):
    return ((cols // 32 * 2) + 15) & ~15


def q4cp_blob_bytes(rows, cols):
    return 64 + rows * cols // 2 + rows * q4cp_scale_stride(cols)


# The 16-entry table the reference's converter writes into every routed-expert tensor unless told otherwise
# (tools/flashnext2hgn.py:530-531, UNIVERSAL_EXPERT_CB): sorted, symmetric, not an affine function of the code.
_UCB_HALF = (0.042080, 0.128362, 0.220943, 0.324402, 0.444132, 0.587296, 0.765293, 1.0)
UNIVERSAL_CODEBOOK = np.array([-v for v in _UCB_HALF[::-1]] + list(_UCB_HALF), np.float32)


def make_q4cp(rng, rows, cols, codebook=None, scale_std=0.01, scales=None, codes=None):
    """Random q4cp blob. scales: fp16 |N(0,1)|*scale_std unless given ([rows][cols/32] float16)."""
    assert cols % 32 == 0
    cb = ZP8_CODEBOOK if codebook is None else np.asarray(codebook, np.float32)
    ss = q4cp_scale_stride(cols)
    blob = np.zeros(q4cp_blob_bytes(rows, cols), np.uint8)
    blob[:64] = cb.view(np.uint8)
    nb = rows * cols // 2
    blob[64:64 + nb] = (rng.integers(0, 256, nb, dtype=np.uint8) if codes is None
                        else np.asarray(codes, np.uint8).reshape(-1))
    if scales is None:
        scales = (np.abs(rng.standard_normal((rows, cols // 32), dtype=np.float32)) * scale_std
                  ).astype(np.float16)
    rec = np.zeros((rows, ss // 2), np.float16)
    rec[:, :cols // 32] = scales
    blob[64 + nb:] = rec.view(np.uint8).reshape(-1)
    return blob


def q4k_row_bytes(cols):
    return cols // 256 * 144


def pack_scale_min_k4(sc, mn):
    """Inverse of get_scale_min_k4: 8 six-bit scales + 8 six-bit mins -> 12 bytes."""
    sc = np.asarray(sc, np.uint8)
    mn = np.asarray(mn, np.uint8)
    q = np.zeros(sc.shape[:-1] + (12,), np.uint8)
    for j in range(4):
        q[..., j] = (sc[..., j] & 63) | ((sc[..., j + 4] >> 4) << 6)
        q[..., j + 4] = (mn[..., j] & 63) | ((mn[..., j + 4] >> 4) << 6)
        q[..., j + 8] = (sc[..., j + 4] & 0xF) | ((mn[..., j + 4] & 0xF) << 4)
    return q


def make_q4k(rng, rows, cols, scale_std=0.01):
    """Random Q4_K rows: d,dmin = fp16(|N(0,1)|*scale_std); sub-scales/mins uniform [0,63]."""
    assert cols % 256 == 0
    nb = rows * cols // 256
    blk = np.zeros((nb, 144), np.uint8)
    dd = (np.abs(rng.standard_normal((nb, 2), dtype=np.float32)) * scale_std).astype(np.float16)
    blk[:, 0:4] = dd.view(np.uint8)
    sc = rng.integers(0, 64, (nb, 8), dtype=np.uint8)
    mn = rng.integers(0, 64, (nb, 8), dtype=np.uint8)
    blk[:, 4:16] = pack_scale_min_k4(sc, mn)
    blk[:, 16:] = rng.integers(0, 256, (nb, 128), dtype=np.uint8)
    return blk.reshape(-1)


def make_q5k(rng, rows, cols, scale_std=0.01):
    """Random Q5_K rows (176-byte super-blocks: d, dmin, scales[12], qh[32], ql[128]; src/gguf.h:408-441)."""
    assert cols % 256 == 0
    nb = rows * cols // 256
    blk = np.zeros((nb, 176), np.uint8)
    dd = (np.abs(rng.standard_normal((nb, 2), dtype=np.float32)) * scale_std).astype(np.float16)
    blk[:, 0:4] = dd.view(np.uint8)
    sc = rng.integers(0, 64, (nb, 8), dtype=np.uint8)
    mn = rng.integers(0, 64, (nb, 8), dtype=np.uint8)
    blk[:, 4:16] = pack_scale_min_k4(sc, mn)
    blk[:, 16:] = rng.integers(0, 256, (nb, 160), dtype=np.uint8)
    return blk.reshape(-1)


def make_q8_0(rng, rows, cols, scale_std=0.01):
    """Random Q8_0 rows (34-byte blocks: d fp16, 32 x int8; src/gguf.h:352-359)."""
    assert cols % 32 == 0
    nb = rows * cols // 32
    blk = np.zeros((nb, 34), np.uint8)
    blk[:, 0:2] = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * scale_std / 8).astype(np.float16).view(np.uint8)
    blk[:, 2:] = rng.integers(0, 256, (nb, 32), dtype=np.uint8)
    return blk.reshape(-1)


def make_q5_1(rng, rows, cols, scale_std=0.01):
    """Random Q5_1 rows (24-byte blocks: d, m fp16, qh u32, qs[16]; src/gguf.h:360-375); m = -16 d so that
    the 5-bit codes are centred like the other formats' weights."""
    assert cols % 32 == 0
    nb = rows * cols // 32
    blk = np.zeros((nb, 24), np.uint8)
    d = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * scale_std / 2).astype(np.float16)
    blk[:, 0:2] = d.view(np.uint8)
    blk[:, 2:4] = (d.astype(np.float32) * -16).astype(np.float16).view(np.uint8)
    blk[:, 4:] = rng.integers(0, 256, (nb, 20), dtype=np.uint8)
    return blk.reshape(-1)


def make_iq4_nl(rng, rows, cols, scale_std=0.01):
    """Random IQ4_NL rows (18-byte blocks: d fp16, qs[16]; codes index a 16-entry table of int8; src/gguf.h:376-388)."""
    assert cols % 32 == 0
    nb = rows * cols // 32
    blk = np.zeros((nb, 18), np.uint8)
    blk[:, 0:2] = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * scale_std / 16).astype(np.float16).view(np.uint8)
    blk[:, 2:] = rng.integers(0, 256, (nb, 16), dtype=np.uint8)
    return blk.reshape(-1)


def make_iq4_xs(rng, rows, cols, scale_std=0.01):
    """Random IQ4_XS rows (136-byte super-blocks: d fp16, scales_h u16, scales_l[4], qs[128]; src/gguf.h:389-407)."""
    assert cols % 256 == 0
    nb = rows * cols // 256
    blk = np.zeros((nb, 136), np.uint8)
    blk[:, 0:2] = (np.abs(rng.standard_normal((nb, 1), dtype=np.float32)) * scale_std / 256).astype(np.float16).view(np.uint8)
    blk[:, 2:] = rng.integers(0, 256, (nb, 134), dtype=np.uint8)
    return blk.reshape(-1)


GG_Q4_K, GG_Q5_K, GG_Q5_1, GG_Q8_0, GG_IQ4_NL, GG_IQ4_XS = 12, 13, 7, 8, 20, 23  # ggml type ids


def make_gg(rng, t, rows, cols, scale_std=0.01):
    return {GG_Q4_K: make_q4k, GG_Q5_K: make_q5k, GG_Q5_1: make_q5_1, GG_Q8_0: make_q8_0, GG_IQ4_NL: make_iq4_nl,
            GG_IQ4_XS: make_iq4_xs}[t](rng, rows, cols, scale_std)


def quantize_q8g64(w):
    """f32 [rows][cols] -> the reference checkpoint format's q8g64 bytes (src/hgn.h:189-196): per row cols uint8
    codes, then cols/64 pairs of fp16 (scale, min), w ~ code * scale + min.  uint8 [rows][cols + cols/64*4]."""
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    assert cols % 64 == 0
    g = w.reshape(rows, cols // 64, 64)
    mn = g.min(axis=2).astype(np.float16)
    sc = ((g.max(axis=2) - mn.astype(np.float32)) / 255.0).astype(np.float16)
    scf = np.where(sc == 0, np.float16(1), sc).astype(np.float32)
    codes = np.clip(np.rint((g - mn.astype(np.float32)[..., None]) / scf[..., None]), 0, 255).astype(np.uint8)
    sm = np.stack([sc, mn], axis=2).reshape(rows, cols // 64 * 2).view(np.uint8)
    return np.ascontiguousarray(np.concatenate([codes.reshape(rows, cols), sm], axis=1))


def make_q8g64(rng, rows, cols, std=0.05):
    return quantize_q8g64(rng.standard_normal((rows, cols), dtype=np.float32) * std)


def quantize_q8g32(w):
    """f32 [rows][cols] -> the reference checkpoint format's planar q8g32 bytes (src/hgn.h:18,176-183): rows*cols int8
    codes, then rows*cols/32 fp16 scales, w ~ code * scale (llama.cpp's Q8_0 arithmetic)."""
    w = np.ascontiguousarray(w, np.float32)
    rows, cols = w.shape
    assert cols % 32 == 0
    g = w.reshape(-1, 32)
    sc = (np.abs(g).max(axis=1) / 127.0).astype(np.float16)
    scf = np.where(sc == 0, np.float16(1), sc).astype(np.float32)
    codes = np.clip(np.rint(g / scf[:, None]), -127, 127).astype(np.int8)
    return np.ascontiguousarray(np.concatenate([codes.reshape(-1).view(np.uint8), sc.view(np.uint8)]))


def make_dense(rng, kind, rows, cols, std=0.05):
    """A dense weight matrix as stored bytes: kind "bf16" (uint16 bit patterns), "f32", "q8g64" or "q8g32"."""
    if kind == "q8g64":
        return make_q8g64(rng, rows, cols, std)
    if kind == "q8g32":
        return quantize_q8g32(rng.standard_normal((rows, cols), dtype=np.float32) * std)
    w = rng.standard_normal((rows, cols), dtype=np.float32) * std
    return f32_to_bf16_bits(w) if kind == "bf16" else w


def make_i4r(rng, rows, cols, scale_std=0.01):
    """hgn v2 i4r tensor (dtype 23): [rows*cols/2 code bytes (byte b = elements 2b | 2b+1 << 4)][rows x cols/128 fp16
    scales], w = (nibble - 8) * scale.  Scales of either sign (the reference's encoder stores signed scales,
    tools/v2repro/v2enc.py:103-106)."""
    assert cols % 128 == 0
    codes = rng.integers(0, 256, size=rows * cols // 2, dtype=np.uint8)
    sc = (rng.standard_normal((rows, cols // 128)) * scale_std).astype(np.float16)
    return np.concatenate([codes, sc.reshape(-1).view(np.uint8)])


def make_v2_planes(rng, d, mid):
    """The four sign-scale planes of an hgn v2 layer's expert tensors as f16-representable f32 values (the files hold
    them as f16): su [d], svh_gu [2 mid], suh_dn [mid], svh_dn [d]; magnitudes near 1, random signs."""
    def plane(n):
        v = (0.5 + rng.random(n)) * rng.choice([-1.0, 1.0], size=n)
        return v.astype(np.float16).astype(np.float32)
    return plane(d), plane(2 * mid), plane(mid), plane(d)


def f32_to_bf16_bits(a):
    """Round-to-nearest-even f32 -> bf16 bit patterns (uint16)."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) >> 16).astype(np.uint16)


def bf16_round(a):
    return (f32_to_bf16_bits(a).astype(np.uint32) << 16).view(np.float32)


def zipf_bias(rng, E, s=1.1, beta=1.0):
    """Per-expert logit bias b_e = -beta*s*ln(rank_e) under a random rank permutation."""
    rank = rng.permutation(E) + 1
    return (-beta * s * np.log(rank)).astype(np.float32)
