"""Full-size synthetic MoE layers generated directly in HBM (torch is only the allocator / RNG).

Byte layouts are the engine's: hgn q4cp blobs and GGUF Q4_K raw blocks.  The checker (tests, benchmark baseline) is fed the
very same bytes, read back from the device, so both sides see identical weights.
"""
import numpy as np
import torch

from . import capi
from . import synth as S


def _gen(seed):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    return g


def q4cp_blob(g, rows, cols, scale_std=0.01, codebook=None):
    """uint8 tensor [64 + rows*cols/2 + rows*ss]: zero-point-8 codebook (or the 16 floats given), uniform codes,
    fp16 |N|*std scales."""
    ss = S.q4cp_scale_stride(cols)
    nb = rows * cols // 2
    blob = torch.empty(64 + nb + rows * ss, dtype=torch.uint8, device="cuda")
    cb = S.ZP8_CODEBOOK if codebook is None else np.ascontiguousarray(codebook, np.float32)
    blob[:64] = torch.from_numpy(cb.view(np.uint8).copy()).cuda()
    step = 1 << 28
    for i in range(0, nb, step):
        n = min(step, nb - i)
        blob[64 + i:64 + i + n] = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    rec = blob[64 + nb:].view(rows, ss)
    rec.zero_()
    G = cols // 32
    crow = max(1, (1 << 26) // G)
    for r0 in range(0, rows, crow):
        r1 = min(rows, r0 + crow)
        sc = (torch.randn((r1 - r0, G), device="cuda", generator=g).abs() * scale_std).to(torch.float16)
        rec[r0:r1, :G * 2] = sc.view(torch.uint8)
    return blob


def i4r_blob(g, rows, cols, scale_std=0.01):
    """uint8 tensor [rows*cols/2 codes][rows x cols/128 fp16 scales] (hgn v2 dtype 23): uniform codes, N*std scales
    of either sign."""
    nb = rows * cols // 2
    blob = torch.empty(nb + rows * (cols // 128) * 2, dtype=torch.uint8, device="cuda")
    step = 1 << 28
    for i in range(0, nb, step):
        n = min(step, nb - i)
        blob[i:i + n] = torch.randint(0, 256, (n,), dtype=torch.uint8, device="cuda", generator=g)
    sc = (torch.randn((rows * (cols // 128),), device="cuda", generator=g) * scale_std).to(torch.float16)
    blob[nb:] = sc.view(torch.uint8)
    return blob


def v2_plane(g, n):
    """A sign-scale plane of an hgn v2 tensor: f16-representable values of magnitude 0.5 .. 1.5, random signs, as f32."""
    v = (0.5 + torch.rand((n,), device="cuda", generator=g)) * (torch.randint(0, 2, (n,), device="cuda", generator=g) * 2 - 1)
    return v.to(torch.float16).to(torch.float32)


def q4k_rows(g, rows, cols, scale_std=0.01):
    """uint8 tensor of rows*cols/256 Q4_K super-blocks (144 B): d,dmin fp16 |N|*std; 6-bit sub-scales/mins
    uniform [0,63]; codes uniform."""
    nb = rows * cols // 256
    blk = torch.empty((nb, 144), dtype=torch.uint8, device="cuda")
    dd = (torch.randn((nb, 2), device="cuda", generator=g).abs() * scale_std).to(torch.float16)
    blk[:, 0:4] = dd.view(torch.uint8)
    sc = torch.randint(0, 64, (nb, 8), dtype=torch.uint8, device="cuda", generator=g)
    mn = torch.randint(0, 64, (nb, 8), dtype=torch.uint8, device="cuda", generator=g)
    q = torch.empty((nb, 12), dtype=torch.uint8, device="cuda")
    for j in range(4):
        q[:, j] = (sc[:, j] & 63) | ((sc[:, j + 4] >> 4) << 6)
        q[:, j + 4] = (mn[:, j] & 63) | ((mn[:, j + 4] >> 4) << 6)
        q[:, j + 8] = (sc[:, j + 4] & 0xF) | ((mn[:, j + 4] & 0xF) << 4)
    blk[:, 4:16] = q
    step = max(1, (1 << 28) // 128)
    for i in range(0, nb, step):
        n = min(step, nb - i)
        blk[i:i + n, 16:] = torch.randint(0, 256, (n, 128), dtype=torch.uint8, device="cuda", generator=g)
    return blk.view(-1)


GG_ROW_BYTES = {12: (256, 144), 13: (256, 176), 8: (32, 34), 7: (32, 24),  # ggml type -> (block elements, bytes)
                20: (32, 18), 23: (256, 136)}


def gg_row_bytes(t, cols):
    be, bb = GG_ROW_BYTES[t]
    return cols // be * bb


def gg_rows(g, t, rows, cols, scale_std=0.01):
    """uint8 tensor of raw rows of ggml type t: Q4_K (12), Q5_K (13), Q8_0 (8), Q5_1 (7), IQ4_NL (20) or IQ4_XS (23);
    integer fields uniform, fp16 fields |N|*std scaled so that weights have the size of the Q4_K ones."""
    if t == 12:
        return q4k_rows(g, rows, cols, scale_std)
    be, bb = GG_ROW_BYTES[t]
    nb = rows * cols // be
    blk = torch.empty((nb, bb), dtype=torch.uint8, device="cuda")
    step = max(1, (1 << 28) // bb)
    for i in range(0, nb, step):
        n = min(step, nb - i)
        blk[i:i + n] = torch.randint(0, 256, (n, bb), dtype=torch.uint8, device="cuda", generator=g)
    if t == 13:    # d, dmin, packed 6-bit scales (any bytes are valid), qh, ql
        dd = (torch.randn((nb, 2), device="cuda", generator=g).abs() * scale_std / 2).to(torch.float16)
        blk[:, 0:4] = dd.view(torch.uint8)
    elif t == 8:   # d, 32 x int8
        dd = (torch.randn((nb, 1), device="cuda", generator=g).abs() * scale_std / 8).to(torch.float16)
        blk[:, 0:2] = dd.view(torch.uint8)
    elif t == 20:  # IQ4_NL: d, 16 code bytes into a table of int8 values up to 127 in size
        dd = (torch.randn((nb, 1), device="cuda", generator=g).abs() * scale_std / 8).to(torch.float16)
        blk[:, 0:2] = dd.view(torch.uint8)
    elif t == 23:  # IQ4_XS: d, 6-bit sub-block scales (minus 32) in scales_h / scales_l, 128 code bytes
        dd = (torch.randn((nb, 1), device="cuda", generator=g).abs() * scale_std / 128).to(torch.float16)
        blk[:, 0:2] = dd.view(torch.uint8)
    else:          # Q5_1: d, m = -16 d, qh, qs
        dd = (torch.randn((nb, 1), device="cuda", generator=g).abs() * scale_std / 2).to(torch.float16)
        blk[:, 0:2] = dd.view(torch.uint8)
        blk[:, 2:4] = (dd.float() * -16).to(torch.float16).view(torch.uint8)
    return blk.view(-1)


class DeviceLayer:
    """One layer's weights in HBM + registration into a capi.Moe context.
    fmt "q4k": raw GGUF blocks, gg_types = ggml types of (gate/up, down, shared expert).
    fmt "i4r": hgn v2 rotated routed experts with their four planes; the shared expert as in a q4cp layer.
    codebook (q4cp): "zp8" = the zero-point-8 grid cb[n] = n - 8; "universal" = the fixed non-uniform table of the
    reference's converter (scales 8.4 times larger, so that the weights keep their size)."""

    def __init__(self, seed, d=3072, mid=768, E=512, k=10, fmt="q4cp", bias=None, gg_types=(12, 12, 12),
                 codebook="zp8"):
        g = _gen(seed)
        self.d, self.mid, self.E, self.k, self.fmt = d, mid, E, k, fmt
        self.tgu, self.tdn, self.tsh = gg_types
        self.router = torch.randn((E, d), device="cuda", generator=g) * 0.02
        self.sh_sg = torch.randn((1, d), device="cuda", generator=g) * 0.02
        self.bias = bias
        if fmt == "q4cp":
            cb, sd = (S.UNIVERSAL_CODEBOOK, 0.084) if codebook == "universal" else (None, 0.01)
            self.gate_up = q4cp_blob(g, E * 2 * mid, d, sd, cb)
            self.down = q4cp_blob(g, E * d, mid, sd, cb)
            self.sh = [q4cp_blob(g, mid, d, sd, cb), q4cp_blob(g, mid, d, sd, cb), q4cp_blob(g, d, mid, sd, cb)]
        elif fmt == "i4r":
            self.gate_up = i4r_blob(g, E * 2 * mid, d)
            self.down = i4r_blob(g, E * d, mid)
            self.planes = [v2_plane(g, d), v2_plane(g, 2 * mid), v2_plane(g, mid), v2_plane(g, d)]
            self.sh = [q4cp_blob(g, mid, d), q4cp_blob(g, mid, d), q4cp_blob(g, d, mid)]
        else:
            self.gate = gg_rows(g, self.tgu, E * mid, d)
            self.up = gg_rows(g, self.tgu, E * mid, d)
            self.down = gg_rows(g, self.tdn, E * d, mid)
            self.sh = [gg_rows(g, self.tsh, mid, d), gg_rows(g, self.tsh, mid, d), gg_rows(g, self.tsh, d, mid)]

    def expert_bytes(self):
        d, mid = self.d, self.mid
        if self.fmt == "q4cp":
            return 2 * mid * (d // 2 + S.q4cp_scale_stride(d)) + d * (mid // 2 + S.q4cp_scale_stride(mid))
        if self.fmt == "i4r":
            return 2 * mid * (d // 2 + d // 128 * 2) + d * (mid // 2 + mid // 128 * 2)
        return 2 * mid * gg_row_bytes(self.tgu, d) + d * gg_row_bytes(self.tdn, mid)

    def shared_bytes(self):
        d, mid = self.d, self.mid
        if self.fmt == "q4cp":
            return self.expert_bytes()
        if self.fmt == "i4r":
            return 2 * mid * (d // 2 + S.q4cp_scale_stride(d)) + d * (mid // 2 + S.q4cp_scale_stride(mid))
        return 2 * mid * gg_row_bytes(self.tsh, d) + d * gg_row_bytes(self.tsh, mid)

    def register(self, m, layer=0):
        d, mid, E = self.d, self.mid, self.E
        m.set_router(layer, capi.wview(self.router, capi.F32, E, d), self.bias)
        if self.fmt == "q4cp":
            m.set_experts_q4cp(layer, capi.wview(self.gate_up, capi.Q4CP, E * 2 * mid, d),
                               capi.wview(self.down, capi.Q4CP, E * d, mid))
            wt, gt = capi.Q4CP, 0
        elif self.fmt == "i4r":
            m.set_experts_i4r(layer, capi.wview(self.gate_up, capi.I4R, E * 2 * mid, d),
                              capi.wview(self.down, capi.I4R, E * d, mid), *self.planes)
            wt, gt = capi.Q4CP, 0
        else:
            m.set_experts_gguf(layer, self.gate, self.up, self.down, self.tgu, self.tdn)
            wt, gt = 0, self.tsh
        m.set_shared(layer, capi.wview(self.sh[0], wt, mid, d), capi.wview(self.sh[1], wt, mid, d),
                     capi.wview(self.sh[2], wt, d, mid), capi.wview(self.sh_sg, capi.F32, 1, d), gt)


def calibrate_zipf(router, x, k, s=1.1, target=12.0, seed=3):
    """Per-expert logit bias b_e = -beta*s*ln(rank_e) (random rank permutation), beta chosen so that the
    hottest expert receives ~target x the mean pair count.  Uses plain torch only to pick beta."""
    E = router.shape[0]
    g = torch.Generator(device="cpu")
    g.manual_seed(seed)
    rank = (torch.randperm(E, generator=g) + 1).to(torch.float32).cuda()
    logits = x @ router.T
    lo, hi = 0.0, 4.0
    for _ in range(20):
        beta = 0.5 * (lo + hi)
        b = -beta * s * torch.log(rank)
        top = torch.topk(logits + b, k, dim=1).indices
        cnt = torch.bincount(top.reshape(-1), minlength=E).float()
        ratio = (cnt.max() / cnt.mean()).item()
        if ratio < target:
            lo = beta
        else:
            hi = beta
    beta = 0.5 * (lo + hi)
    return (-beta * s * torch.log(rank)).contiguous(), beta


def verify_batch(router, d, T=20, share=0.3, k=10, seed=5):
    """Activations for a speculative-verify batch: ~share of the tokens are small perturbations of a
    template token, so their router logits reproduce its top-k set."""
    g = _gen(seed)
    x = torch.randn((T, d), device="cuda", generator=g)
    n = int(round(share * T))
    for i in range(1, n):
        x[i] = x[0] + 1e-3 * torch.randn((d,), device="cuda", generator=g)
    return x
