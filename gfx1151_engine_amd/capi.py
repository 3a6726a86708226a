"""ctypes binding of libmi355moe.so (include/mi355_moe.h).

PyTorch supplies device memory and the stream only; every computation is a call through the
C ABI.  Loading fails loudly when the library has not been built — there is no fallback path.
"""
import ctypes as C
import os

import torch

from .build import LIB

F32, BF16, Q4CP, Q8G64, Q8G32 = 1, 0, 5, 7, 8
I4R = 23  # hgn v2 routed experts
HT, Q6G64 = 16, 24  # hgn v2 dense tensors (converted to bf16 by v2_dense_to_bf16 / the file loader)
GGML_Q4_K = 12
GGML_Q5_K, GGML_Q5_1, GGML_Q8_0 = 13, 7, 8


class MoeError(RuntimeError):
    pass


class WView(C.Structure):
    _fields_ = [("dtype", C.c_int), ("data", C.c_void_p), ("rows", C.c_uint64), ("cols", C.c_uint64),
                ("scale_stride", C.c_uint64)]


class GgExperts(C.Structure):
    _fields_ = [("gate", C.c_void_p), ("up", C.c_void_p), ("down", C.c_void_p), ("tgu", C.c_int),
                ("tdn", C.c_int)]


class Config(C.Structure):
    _fields_ = [("d", C.c_int), ("mid", C.c_int), ("experts", C.c_int), ("topk", C.c_int),
                ("layers", C.c_int), ("max_tokens", C.c_int), ("id_stride", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        path = os.environ.get("MI355MOE_LIB", LIB)  # another build of the same library (A/B timing runs)
        if not os.path.exists(path):
            raise MoeError(f"{path} is missing: run `python -c 'import __graft_entry__ as g; g.build()'`")
        _lib = C.CDLL(path)
        _lib.moe_version.restype = C.c_char_p
        _lib.moe_status_string.restype = C.c_char_p
    return _lib


def second_binding(path):
    """Another instance of this module, bound to another build of the library at `path` (the benchmark's timing twin):
    its own library handle, the same classes and helpers.  Device pointers are process-wide, so contexts of both
    bindings can work on the same weights."""
    import importlib.util
    if not os.path.exists(path):
        raise MoeError(f"{path} is missing")
    spec = importlib.util.find_spec(__name__)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod._lib = C.CDLL(path)
    mod._lib.moe_version.restype = C.c_char_p
    mod._lib.moe_status_string.restype = C.c_char_p
    return mod


def check(rc, what=""):
    if rc != 0:
        raise MoeError(f"{what}: status {rc} ({lib().moe_status_string(C.c_int(rc)).decode()})")


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else None


def q4cp_scale_stride(cols):
    return ((cols // 32 * 2) + 15) & ~15


def wview(t, dtype, rows, cols):
    """A weight tensor (torch uint8 / float32 / bfloat16 on the GPU) as the engine's WView."""
    ss = q4cp_scale_stride(cols) if dtype == Q4CP else 0
    v = WView(dtype, t.data_ptr(), rows, cols, ss)
    v._keep = t
    return v


def u64(v):
    return C.c_uint64(int(v))


# ---- stage-level calls ----

def q4cp_dequant_rows(blob, rows, cols, row0, nrows):
    out = torch.empty((nrows, cols), dtype=torch.float32, device=blob.device)
    check(lib().moe_q4cp_dequant_rows(ptr(blob), u64(rows), u64(cols), u64(row0), u64(nrows), ptr(out),
                                      stream()), "moe_q4cp_dequant_rows")
    return out


def q4k_dequant_rows(raw, nrows, cols):
    out = torch.empty((nrows, cols), dtype=torch.float32, device=raw.device)
    check(lib().moe_q4k_dequant_rows(ptr(raw), u64(nrows), u64(cols), ptr(out), stream()),
          "moe_q4k_dequant_rows")
    return out


def gg_dequant_rows(gtype, raw, nrows, cols):
    out = torch.empty((nrows, cols), dtype=torch.float32, device=raw.device)
    check(lib().moe_gg_dequant_rows(gtype, ptr(raw), u64(nrows), u64(cols), ptr(out), stream()),
          "moe_gg_dequant_rows")
    return out


def router_logits(W, x, bias=None, mode=0):
    P = x.shape[0]
    out = torch.empty((P, W.rows), dtype=torch.float32, device=x.device)
    check(lib().moe_router_logits(C.byref(W), ptr(bias), ptr(x), P, ptr(out), mode, stream()),
          "moe_router_logits")
    return out


def router_topk(logits, k, id_stride=16):
    P, E = logits.shape
    ids = torch.zeros((P, id_stride), dtype=torch.int32, device=logits.device)
    ws = torch.zeros((P, id_stride), dtype=torch.float32, device=logits.device)
    check(lib().moe_router_topk(ptr(logits), ptr(ids), ptr(ws), P, E, k, id_stride, stream()),
          "moe_router_topk")
    return ids, ws


class Routing:
    """GpuMoeRouting: init(capacity, experts) / run(...)."""

    def __init__(self, capacity_pairs, experts):
        self.h = C.c_void_p()
        self.experts = experts
        check(lib().moe_routing_create(capacity_pairs, experts, C.byref(self.h)), "moe_routing_create")

    def run(self, ids, ws, k, want_pairids=True):
        P, stride = ids.shape
        dev = ids.device
        n = P * k
        tokidx = torch.full((max(n, 1),), -1, dtype=torch.int32, device=dev)
        pw = torch.zeros((max(n, 1),), dtype=torch.float32, device=dev)
        eoff = torch.full((self.experts + 1,), -1, dtype=torch.int32, device=dev)
        pairids = torch.full((max(n, 1),), -1, dtype=torch.int32, device=dev) if want_pairids else None
        check(lib().moe_routing_run(self.h, ptr(ids), ptr(ws), ptr(tokidx), ptr(pw), ptr(eoff), ptr(pairids),
                                    P, k, self.experts, stride, stream()), "moe_routing_run")
        return tokidx[:n], pw[:n], eoff, (pairids[:n] if want_pairids else None)

    def close(self):
        if self.h:
            check(lib().moe_routing_destroy(self.h), "moe_routing_destroy")
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def routing_run_static(ids, ws, k, experts, want_pairids=True):
    """moe_routing_run_static: the permutation on the library's fixed scratch (the outputs are the caller's)."""
    P, stride = ids.shape
    dev = ids.device
    n = P * k
    tokidx = torch.full((max(n, 1),), -1, dtype=torch.int32, device=dev)
    pw = torch.zeros((max(n, 1),), dtype=torch.float32, device=dev)
    eoff = torch.full((experts + 1,), -1, dtype=torch.int32, device=dev)
    pairids = torch.full((max(n, 1),), -1, dtype=torch.int32, device=dev) if want_pairids else None
    check(lib().moe_routing_run_static(ptr(ids), ptr(ws), ptr(tokidx), ptr(pw), ptr(eoff), ptr(pairids), P, k,
                                       experts, stride, stream()), "moe_routing_run_static")
    return tokidx[:n], pw[:n], eoff, (pairids[:n] if want_pairids else None)


def tiles(eoff, cap, pairs):
    E = eoff.numel() - 1
    max_tiles = (pairs + cap - 1) // cap + E
    t = torch.zeros((max_tiles, 3), dtype=torch.int32, device=eoff.device)
    n = torch.zeros((1,), dtype=torch.int32, device=eoff.device)
    check(lib().moe_tiles(ptr(eoff), ptr(t), ptr(n), E, cap, stream()), "moe_tiles")
    return t, n


def q4cp_gemv_gate_up(gu, x, ids, kpt, mid):
    P = x.shape[0]
    hid = torch.empty((P * kpt, mid), dtype=torch.float32, device=x.device)
    check(lib().moe_q4cp_gemv_gate_up(C.byref(gu), ptr(x), u64(x.stride(0)), ptr(ids), ids.shape[1], kpt, P,
                                      mid, ptr(hid), stream()), "moe_q4cp_gemv_gate_up")
    return hid


def q4cp_gemv_down_topk(dn, hid, ids, ws, kpt, d, ey=None, sg=None):
    P = ids.shape[0]
    out = torch.empty((P, d), dtype=torch.float32, device=hid.device)
    check(lib().moe_q4cp_gemv_down_topk(C.byref(dn), ptr(hid), ptr(ids), ptr(ws), ids.shape[1], kpt, P, d,
                                        ptr(ey), ptr(sg), ptr(out), u64(d), stream()),
          "moe_q4cp_gemv_down_topk")
    return out


class LutW(C.Structure):
    _fields_ = [("w", C.c_void_p), ("w_up", C.c_void_p), ("sc", C.c_void_p), ("sc_up", C.c_void_p),
                ("cb", C.c_void_p), ("sstride", C.c_int), ("e_rows", C.c_int), ("up_off", C.c_int)]


LUT_Q4CP = 100
LUT_I4R = 101
ROUTING_STATIC_MAX_TOKENS = 32768
DENSE_SHARED = True  # moe_set_shared takes bf16 / f32 / q8g64 matrices
OPT_INT_DECODE = 1
OPT_UNIQUE_MIN_TOKENS = 2
OPT_FUSED_COMBINE = 3
OPT_SHARED_ASIDE = 4
OPT_TIMING_SKIP_STAGE = 5
OPT_ROUTER_CANDIDATES = 6
OPT_UNIQUE_GGUF = 7
OPT_GU_TOPK_MAX_TOKENS = 8
OPT_F32_DECODE_MAX_TOKENS = 9
OPT_V2_FUSED_MIDDLE = 10
OPT_PAIR_TABLES = 11
PATH_NONE, PATH_SMALL, PATH_BATCH, PATH_WALKED = 0, 1, 2, 3


def lut_q4cp_view(blob, rows, cols, e_rows, up_off):
    p = LutW()
    check(lib().moe_lut_q4cp_view(ptr(blob), u64(rows), u64(cols), u64(0), e_rows, up_off, C.byref(p)),
          "moe_lut_q4cp_view")
    p._keep = blob
    return p


def lut_i4r_view(blob, rows, cols, e_rows, up_off=0):
    p = LutW()
    check(lib().moe_lut_i4r_view(ptr(blob), u64(rows), u64(cols), e_rows, up_off, C.byref(p)), "moe_lut_i4r_view")
    p._keep = blob
    return p


def i4r_dequant_rows(blob, rows, cols, row0, nrows):
    out = torch.empty((nrows, cols), dtype=torch.float32, device=blob.device)
    check(lib().moe_i4r_dequant_rows(ptr(blob), u64(rows), u64(cols), u64(row0), u64(nrows), ptr(out), stream()),
          "moe_i4r_dequant_rows")
    return out


def v2_dense_to_bf16(dtype, blob, rows, cols, suh=None, svh=None):
    """An hgn v2 dense tensor (HT with its planes as f32, or Q6G64) -> the bf16 bits [rows][cols] of the matrix."""
    out = torch.empty((rows, cols), dtype=torch.int16, device=blob.device)
    check(lib().moe_v2_dense_to_bf16(dtype, ptr(blob), ptr(suh), ptr(svh), u64(rows), u64(cols), ptr(out), stream()),
          "moe_v2_dense_to_bf16")
    return out


def v2_rot(x, pre=None, post=None, out_f16=False):
    """post * H(pre * x) / sqrt(128) per 128 block of every row; f32 rows, or f16 rows in layout 1."""
    P, n = x.shape
    y = torch.empty((P, n), dtype=torch.float16 if out_f16 else torch.float32, device=x.device)
    check(lib().moe_v2_rot(ptr(x), u64(n), ptr(y), u64(n), ptr(pre), ptr(post), n, P, 1 if out_f16 else 0, stream()),
          "moe_v2_rot")
    return y


def i4r_mid(guv, svh_gu, suh_dn, mid, out_f16=False):
    """guv [nslots][2 mid] (f32 or f16) -> the rotated down-projection input [nslots][mid] (f32, or f16 in layout 1)."""
    n = guv.shape[0]
    out = torch.empty((n, mid), dtype=torch.float16 if out_f16 else torch.float32, device=guv.device)
    check(lib().moe_i4r_mid(ptr(guv), 1 if guv.dtype == torch.float16 else 0, u64(guv.shape[1]), ptr(out),
                            1 if out_f16 else 0, u64(mid), ptr(svh_gu), ptr(suh_dn), mid, n, stream()), "moe_i4r_mid")
    return out


def lut_up_raw(p, x16, tokidx, tiles_t, ntiles, mid, npairs):
    guv = torch.full((npairs, 2 * mid), float("nan"), dtype=torch.float16, device=x16.device)
    check(lib().moe_lut_up_raw(LUT_I4R, C.byref(p), ptr(x16), ptr(tokidx), ptr(tiles_t), ptr(ntiles), tiles_t.shape[0],
                               ptr(guv), mid, x16.shape[1], stream()), "moe_lut_up_raw")
    return guv


def v2_reduce_rot(pairs, pairids, pw, svh, P, K, ey=None, sg=None):
    D = pairs.shape[1]
    out = torch.empty((P, D), dtype=torch.float32, device=pairs.device)
    check(lib().moe_v2_reduce_rot(ptr(pairs), 1 if pairs.dtype == torch.float16 else 0, ptr(pairids), ptr(pw), ptr(svh),
                                  ptr(ey), ptr(sg), ptr(out), P, D, K, stream()), "moe_v2_reduce_rot")
    return out


def f32_to_f16(x, layout=1):
    out = torch.empty(x.shape, dtype=torch.float16, device=x.device)
    check(lib().moe_f32_to_f16(ptr(x), ptr(out), u64(x.numel()), layout, stream()), "moe_f32_to_f16")
    return out


ILV = [0, 4, 1, 5, 2, 6, 3, 7]  # layout 1: position p of a group of 8 holds element ILV[p]


def from_layout1(t):
    """Undo the interleaved f16 activation order (last dim, groups of 8) -> natural order."""
    inv = [ILV.index(e) for e in range(8)]
    s = t.shape
    return t.reshape(*s[:-1], s[-1] // 8, 8)[..., inv].reshape(s)


def _q4k_order():
    o = []
    for w in range(8):
        o += [4 * w, 4 * w + 2, 32 + 4 * w, 32 + 4 * w + 2, 4 * w + 1, 4 * w + 3, 32 + 4 * w + 1, 32 + 4 * w + 3]
    return o


Q4K_ORDER = _q4k_order()  # layout 2: position p of a block of 64 holds element Q4K_ORDER[p]


def from_layout2(t):
    """Undo the Q4_K activation order (last dim, blocks of 64) -> natural order."""
    inv = [Q4K_ORDER.index(e) for e in range(64)]
    s = t.shape
    return t.reshape(*s[:-1], s[-1] // 64, 64)[..., inv].reshape(s)


def gg_up(gate, up, x16, tokidx, tiles_t, ntiles, mid, npairs):
    hid = torch.full((npairs, mid), float("nan"), dtype=torch.float16, device=x16.device)
    check(lib().moe_gg_up(GGML_Q4_K, ptr(gate), ptr(up), ptr(x16), ptr(tokidx), ptr(tiles_t), ptr(ntiles),
                          tiles_t.shape[0], ptr(hid), mid, x16.shape[1], stream()), "moe_gg_up")
    return hid


def gg_down(down, hid16, tiles_t, ntiles, d, f16=True):
    npairs = hid16.shape[0]
    pairs = torch.full((npairs, d), float("nan"), dtype=torch.float16 if f16 else torch.float32,
                       device=hid16.device)
    check(lib().moe_gg_down(GGML_Q4_K, ptr(down), ptr(hid16), ptr(tiles_t), ptr(ntiles), tiles_t.shape[0],
                            ptr(pairs), d, hid16.shape[1], 1 if f16 else 0, stream()), "moe_gg_down")
    return pairs


def lut_up(p, x16, tokidx, tiles_t, ntiles, mid, npairs):
    hid = torch.full((npairs, mid), float("nan"), dtype=torch.float16, device=x16.device)
    check(lib().moe_lut_up(LUT_Q4CP, C.byref(p), ptr(x16), ptr(tokidx), ptr(tiles_t), ptr(ntiles),
                           tiles_t.shape[0], ptr(hid), mid, x16.shape[1], stream()), "moe_lut_up")
    return hid


def lut_down(p, hid16, tiles_t, ntiles, d, f16=True, lut_type=LUT_Q4CP):
    npairs = hid16.shape[0]
    pairs = torch.full((npairs, d), float("nan"), dtype=torch.float16 if f16 else torch.float32,
                       device=hid16.device)
    check(lib().moe_lut_down(lut_type, C.byref(p), ptr(hid16), ptr(tiles_t), ptr(ntiles), tiles_t.shape[0],
                             ptr(pairs), d, hid16.shape[1], 1 if f16 else 0, stream()), "moe_lut_down")
    return pairs


def reduce_pw_sg(pairs, pairids, pw, P, K, ey=None, sg=None):
    D = pairs.shape[1]
    out = torch.empty((P, D), dtype=torch.float32, device=pairs.device)
    check(lib().moe_reduce_pw_sg(ptr(pairs), 1 if pairs.dtype == torch.float16 else 0, ptr(pairids), ptr(pw),
                                 ptr(ey), ptr(sg), ptr(out), P, D, K, stream()), "moe_reduce_pw_sg")
    return out


def reduce_pw_sg_hc(pairs, pairids, pw, P, K, w4, R, ey=None, sg=None):
    D = pairs.shape[1]
    check(lib().moe_reduce_pw_sg_hc(ptr(pairs), 1 if pairs.dtype == torch.float16 else 0, ptr(pairids), ptr(pw),
                                    ptr(ey), ptr(sg), ptr(w4), ptr(R), P, D, K, stream()), "moe_reduce_pw_sg_hc")
    return R


# ---- model level ----

class Moe:
    """moe_ctx: weights are borrowed torch tensors (kept alive here), scratch lives in the context."""

    def __init__(self, d, mid, experts, topk, layers=1, max_tokens=32, id_stride=16):
        self.cfg = Config(d, mid, experts, topk, layers, max_tokens, id_stride)
        self.h = C.c_void_p()
        self._keep = []
        check(lib().moe_create(C.byref(self.cfg), C.byref(self.h)), "moe_create")

    def set_router(self, layer, W, bias=None):
        self._keep += [W, bias]
        check(lib().moe_set_router(self.h, layer, C.byref(W), ptr(bias)), "moe_set_router")

    def set_experts_q4cp(self, layer, gate_up, down):
        self._keep += [gate_up, down]
        check(lib().moe_set_experts_q4cp(self.h, layer, C.byref(gate_up), C.byref(down)),
              "moe_set_experts_q4cp")

    def set_experts_i4r(self, layer, gate_up, down, su, svh_gu, suh_dn, svh_dn):
        """hgn v2 routed experts: I4R views and the four sign-scale planes as f32 device tensors."""
        self._keep += [gate_up, down, su, svh_gu, suh_dn, svh_dn]
        check(lib().moe_set_experts_i4r(self.h, layer, C.byref(gate_up), C.byref(down), ptr(su), ptr(svh_gu),
                                        ptr(suh_dn), ptr(svh_dn)), "moe_set_experts_i4r")

    def set_experts_gguf(self, layer, gate, up, down, tgu=GGML_Q4_K, tdn=GGML_Q4_K):
        self._keep += [gate, up, down]
        gg = GgExperts(gate.data_ptr(), up.data_ptr(), down.data_ptr(), tgu, tdn)
        check(lib().moe_set_experts_gguf(self.h, layer, C.byref(gg)), "moe_set_experts_gguf")

    def set_shared(self, layer, gate_proj, up_proj, down_proj, shared_gate, gguf_type=0):
        self._keep += [gate_proj, up_proj, down_proj, shared_gate]
        check(lib().moe_set_shared(self.h, layer, C.byref(gate_proj), C.byref(up_proj), C.byref(down_proj),
                                   C.byref(shared_gate), gguf_type), "moe_set_shared")

    def forward(self, layer, x, y=None):
        P = x.shape[0]
        if y is None:
            y = torch.empty((P, self.cfg.d), dtype=torch.float32, device=x.device)
        check(lib().moe_forward(self.h, layer, ptr(x), P, ptr(y), stream()), "moe_forward")
        return y

    def forward_x16(self, layer, x, x16, y=None):
        """moe_forward_x16: the caller's f16 copy of x (capi.f32_to_f16(x, layout=self.x16_layout(layer)))."""
        P = x.shape[0]
        if y is None:
            y = torch.empty((P, self.cfg.d), dtype=torch.float32, device=x.device)
        check(lib().moe_forward_x16(self.h, layer, ptr(x), ptr(x16), P, ptr(y), stream()), "moe_forward_x16")
        return y

    def x16_layout(self, layer):
        rc = lib().moe_x16_layout(self.h, layer)
        if rc < 0:
            check(rc, "moe_x16_layout")
        return rc

    def forward_hc(self, layer, x, w4, R):
        """moe_b(try_hcw): the combine writes into the bf16 HC state R [P][4][d] (int16 tensor of bf16 bits)."""
        check(lib().moe_forward_hc(self.h, layer, ptr(x), x.shape[0], ptr(w4), ptr(R), stream()), "moe_forward_hc")
        return R

    def set_option(self, option, value):
        check(lib().moe_set_option(self.h, option, value), "moe_set_option")

    def last_path(self):
        """PATH_SMALL / PATH_BATCH / PATH_WALKED of the last forward call (moe_last_path)."""
        return int(lib().moe_last_path(self.h))

    def profile(self, on=True):
        check(lib().moe_profile_enable(self.h, 1 if on else 0), "moe_profile_enable")

    def profile_read(self):
        """-> dict stage -> ms of the last forward (router, route, up, down, reduce)."""
        ms = (C.c_float * 5)()
        check(lib().moe_profile_read(self.h, ms), "moe_profile_read")
        return dict(zip(("router", "route", "up", "down", "reduce"), [float(v) for v in ms]))

    def last_routing(self, P):
        S = self.cfg.id_stride
        ids = torch.empty((P, S), dtype=torch.int32, device="cuda")
        ws = torch.empty((P, S), dtype=torch.float32, device="cuda")
        check(lib().moe_get_routing(self.h, P, ptr(ids), ptr(ws), stream()), "moe_get_routing")
        return ids, ws

    def close(self):
        if self.h:
            check(lib().moe_destroy(self.h), "moe_destroy")
            self.h = C.c_void_p()

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


# ---- checkpoint files ----

class TensorInfo(C.Structure):
    _fields_ = [("dtype", C.c_int), ("ndims", C.c_uint32), ("dims", C.c_uint64 * 4), ("data", C.c_void_p),
                ("nbytes", C.c_uint64)]


FILE_HGN, FILE_GGUF = 1, 2
FILE_OPT_GGUF_F32_ROUTER = 1


class ModelFile:
    """moe_file: a .hgn or GGUF file mapped read-only (host only, no GPU needed)."""

    def __init__(self, path):
        self.h = C.c_void_p()
        check(lib().moe_file_open(str(path).encode(), C.byref(self.h)), f"moe_file_open({path})")

    @property
    def format(self):
        return lib().moe_file_format(self.h)

    def __len__(self):
        lib().moe_file_tensor_count.restype = C.c_int64
        return lib().moe_file_tensor_count(self.h)

    def find(self, name):
        """-> (dtype, dims tuple, bytes as a numpy uint8 copy) or None"""
        import numpy as np
        ti = TensorInfo()
        rc = lib().moe_file_find(self.h, name.encode(), C.byref(ti))
        if rc == -3:
            return None
        check(rc, "moe_file_find")
        data = np.ctypeslib.as_array(C.cast(ti.data, C.POINTER(C.c_uint8)), shape=(ti.nbytes,)).copy() if ti.nbytes else \
            np.zeros(0, np.uint8)
        return ti.dtype, tuple(ti.dims[i] for i in range(ti.ndims)), data

    def set_option(self, option, value):
        check(lib().moe_file_set_option(self.h, option, value), "moe_file_set_option")

    def add_overlay(self, path):
        """True if the overlay file was applied, False if it was left out (already mapped / would replace v2 tensors)."""
        rc = lib().moe_file_add_overlay(self.h, str(path).encode())
        if rc == -3:
            return False
        check(rc, f"moe_file_add_overlay({path})")
        return True

    def config(self, layer=0):
        cfg = Config()
        check(lib().moe_file_config(self.h, layer, C.byref(cfg)), "moe_file_config")
        return cfg

    def load_mtp_layers(self, moe, mtp_layer0, ctx_layer0, n_layers):
        w = C.c_void_p()
        check(lib().moe_load_mtp_layers(moe.h, self.h, mtp_layer0, ctx_layer0, n_layers, C.byref(w), stream()),
              "moe_load_mtp_layers")
        return Weights(w)

    def load_layers(self, moe, file_layer0, ctx_layer0, n_layers):
        """-> opaque weights handle (keep it alive as long as the context uses the layers)"""
        w = C.c_void_p()
        check(lib().moe_load_layers(moe.h, self.h, file_layer0, ctx_layer0, n_layers, C.byref(w), stream()),
              "moe_load_layers")
        return Weights(w)

    def close(self):
        if self.h:
            lib().moe_file_close(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


class Weights:
    def __init__(self, h):
        self.h = h

    @property
    def nbytes(self):
        lib().moe_weights_bytes.restype = C.c_uint64
        return lib().moe_weights_bytes(self.h)

    def free(self):
        if self.h:
            check(lib().moe_weights_free(self.h), "moe_weights_free")
            self.h = None

