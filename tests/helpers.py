"""Shared builders for the tests: seeded layers in the engine's byte layouts, for the oracle
(numpy) and for the HIP library (torch tensors on the GPU) from the same bytes."""
import numpy as np

from gfx1151_engine_amd import synth as S
from oracle import oracle as O


def bits(a):
    return np.ascontiguousarray(a, np.float32).view(np.uint32)


def max_abs_rel(y, ref):
    """max |y - ref| / max |ref|: the layer tolerance is stated on this number."""
    return float(np.abs(y.astype(np.float64) - ref.astype(np.float64)).max() / np.abs(ref).max())


class HostLayer:
    """One synthetic MoE layer as host bytes (the 'file' side)."""

    def __init__(self, rng, d, mid, E, k, fmt="q4cp", router_dtype="f32", codebook=None, scale_std=0.01,
                 router_std=0.02, shared=True, bias=None, gg_types=(12, 12, 12), shared_codebooks=None,
                 shared_dense=None):
        """fmt "q4k": raw GGUF blocks; gg_types = ggml types of (gate/up, down, shared expert).
        shared_codebooks: three 16-entry tables for the shared expert's gate_proj / up_proj / down_proj (q4cp; the
        reference's converter trains one codebook per dense tensor, tools/flashnext2hgn.py:164-187).
        shared_dense: "bf16" / "f32" / "q8g64": the shared expert's matrices in that dense storage instead."""
        self.shared_dense = shared_dense
        self.d, self.mid, self.E, self.k, self.fmt = d, mid, E, k, fmt
        self.tgu, self.tdn, self.tsh = gg_types
        rw = (rng.standard_normal((E, d), dtype=np.float32) * router_std)
        if router_dtype == "bf16":
            self.router = S.f32_to_bf16_bits(rw)
            self.router_dt = O.BF16
        else:
            self.router = rw
            self.router_dt = O.F32
        self.bias = bias
        self.planes = None
        if fmt == "q4cp":
            self.gate_up = S.make_q4cp(rng, E * 2 * mid, d, codebook=codebook, scale_std=scale_std)
            self.down = S.make_q4cp(rng, E * d, mid, codebook=codebook, scale_std=scale_std)
        elif fmt == "i4r":  # hgn v2 rotated experts (the shared expert as in a q4cp layer)
            self.gate_up = S.make_i4r(rng, E * 2 * mid, d, scale_std=scale_std)
            self.down = S.make_i4r(rng, E * d, mid, scale_std=scale_std)
            self.planes = S.make_v2_planes(rng, d, mid)
        else:
            self.gate = S.make_gg(rng, self.tgu, E * mid, d, scale_std=scale_std)
            self.up = S.make_gg(rng, self.tgu, E * mid, d, scale_std=scale_std)
            self.down = S.make_gg(rng, self.tdn, E * d, mid, scale_std=scale_std)
        self.shared = None
        if shared:
            scb = shared_codebooks if shared_codebooks is not None else [codebook] * 3
            mk = (lambda r, c, i: S.make_q4cp(rng, r, c, codebook=scb[i], scale_std=scale_std)) if fmt in ("q4cp", "i4r") \
                else (lambda r, c, i: S.make_gg(rng, self.tsh, r, c, scale_std=scale_std))
            if shared_dense:
                mk = lambda r, c, i: S.make_dense(rng, shared_dense, r, c, std=0.05)
            self.shared = [mk(mid, d, 0), mk(mid, d, 1), mk(d, mid, 2),
                           rng.standard_normal((1, d), dtype=np.float32) * router_std]

    def oracle_layer(self):
        d, mid, E, k = self.d, self.mid, self.E, self.k
        wt = O.Q4CP if self.fmt == "q4cp" else O.I4R if self.fmt == "i4r" else O.Q4K
        sh = None
        if self.shared is not None:
            st = O.Q4CP if self.fmt in ("q4cp", "i4r") else self.tsh
            if self.shared_dense:
                st = {"bf16": O.BF16, "f32": O.F32, "q8g64": O.Q8G64, "q8g32": O.Q8G32}[self.shared_dense]
            sh = [O.Mat(st, self.shared[0], mid, d), O.Mat(st, self.shared[1], mid, d),
                  O.Mat(st, self.shared[2], d, mid), O.Mat(O.F32, self.shared[3], 1, d)]
        router = O.Mat(self.router_dt, self.router, E, d)
        if self.fmt in ("q4cp", "i4r"):
            return O.Layer(d, mid, E, k, router, O.Mat(wt, self.down, E * d, mid),
                           gate_up=O.Mat(wt, self.gate_up, E * 2 * mid, d), shared=sh, router_bias=self.bias,
                           rot=self.planes)
        return O.Layer(d, mid, E, k, router, O.Mat(self.tdn, self.down, E * d, mid),
                       gate=O.Mat(self.tgu, self.gate, E * mid, d), up=O.Mat(self.tgu, self.up, E * mid, d), shared=sh,
                       router_bias=self.bias)

    def to_gpu(self, max_tokens=32, binding=None):
        """-> (capi.Moe context with this layer registered as layer 0, dict of device tensors).
        binding: another binding of the C ABI (capi.second_binding) instead of the default library's."""
        import torch
        from gfx1151_engine_amd import capi
        if binding is not None:
            capi = binding
        d, mid, E, k = self.d, self.mid, self.E, self.k
        dev = {}

        def up(name, a):
            t = torch.from_numpy(np.ascontiguousarray(a)).cuda()
            dev[name] = t
            return t
        m = capi.Moe(d, mid, E, k, layers=1, max_tokens=max_tokens)
        rt = up("router", self.router.view(np.int16) if self.router_dt == O.BF16 else self.router)
        m.set_router(0, capi.wview(rt, capi.BF16 if self.router_dt == O.BF16 else capi.F32, E, d),
                     up("bias", self.bias) if self.bias is not None else None)
        if self.fmt == "q4cp":
            m.set_experts_q4cp(0, capi.wview(up("gate_up", self.gate_up), capi.Q4CP, E * 2 * mid, d),
                               capi.wview(up("down", self.down), capi.Q4CP, E * d, mid))
        elif self.fmt == "i4r":
            m.set_experts_i4r(0, capi.wview(up("gate_up", self.gate_up), capi.I4R, E * 2 * mid, d),
                              capi.wview(up("down", self.down), capi.I4R, E * d, mid),
                              *(up("plane%d" % i, a) for i, a in enumerate(self.planes)))
        else:
            m.set_experts_gguf(0, up("gate", self.gate), up("up", self.up), up("down", self.down), self.tgu, self.tdn)
        if self.shared is not None:
            wt = capi.Q4CP if self.fmt in ("q4cp", "i4r") else 0
            shw = self.shared[:3]
            if self.shared_dense:
                wt = {"bf16": capi.BF16, "f32": capi.F32, "q8g64": capi.Q8G64, "q8g32": capi.Q8G32}[self.shared_dense]
                if self.shared_dense == "bf16":
                    shw = [a.view(np.int16) for a in shw]
            m.set_shared(0, capi.wview(up("shg", shw[0]), wt, mid, d),
                         capi.wview(up("shu", shw[1]), wt, mid, d),
                         capi.wview(up("shd", shw[2]), wt, d, mid),
                         capi.wview(up("shsg", self.shared[3]), capi.F32, 1, d),
                         0 if self.fmt in ("q4cp", "i4r") or self.shared_dense else self.tsh)
        return m, dev
