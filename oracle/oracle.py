"""ctypes binding of oracle/libmoe_oracle.so and (when built) oracle/_ref/libmoe_ref.so.

TEST INFRASTRUCTURE ONLY: the checker for the HIP path, never the thing shipped or measured
(except as bench.py's labelled cpu_baseline).  numpy arrays in, numpy arrays out.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
F32, BF16, Q4CP, Q4K = 1, 0, 5, 12
Q5K, Q5_1, Q8_0, IQ4_NL, IQ4_XS = 13, 7, 8, 20, 23   # further ggml block types of the expert tensors (ids as in GGUF)
Q8G64 = 107  # hgn dtype 7 (the oracle's tag is moved off ggml's Q5_1 = 7)
Q8G32 = 108  # hgn dtype 8 (moved off ggml's Q8_0 = 8)
I4R = 123    # hgn v2 dtype 23 (moved off ggml's IQ4_XS = 23)
HGN_DTYPE = {BF16: 0, F32: 1, Q4CP: 5, Q8G64: 7, Q8G32: 8, I4R: 23}  # oracle tag -> dtype field of the reference's checkpoint format
GG_TYPES = (Q4K, Q5K, Q5_1, Q8_0, IQ4_NL, IQ4_XS)


def build(force=False):
    """Compile the oracle (and the reference shim when /root/reference exists)."""
    args = ["make", "-C", _HERE] + (["-B"] if force else [])
    subprocess.run(args, check=True, stdout=subprocess.DEVNULL)


class _Mat(C.Structure):
    _fields_ = [("dtype", C.c_int), ("data", C.c_void_p), ("rows", C.c_uint64), ("cols", C.c_uint64)]


class _Layer(C.Structure):
    _fields_ = [("d", C.c_int), ("mid", C.c_int), ("E", C.c_int), ("k", C.c_int),
                ("router", _Mat), ("router_bias", C.c_void_p),
                ("gate_up", _Mat), ("gate", _Mat), ("up", _Mat), ("down", _Mat),
                ("sh_gate", _Mat), ("sh_up", _Mat), ("sh_down", _Mat), ("sh_sg", _Mat),
                ("has_shared", C.c_int),
                ("su_gu", C.c_void_p), ("svh_gu", C.c_void_p), ("suh_dn", C.c_void_p), ("svh_dn", C.c_void_p)]


_lib = None
_ref = None


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "libmoe_oracle.so")
        if not os.path.exists(path):
            build()
        _lib = C.CDLL(path)
        _lib.orc_fp16_to_f32.restype = C.c_float
        _lib.orc_fp16_to_f32.argtypes = [C.c_uint16]
        _lib.orc_mat_rows.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_void_p]
        _lib.orc_mat_rows.restype = None
        _lib.orc_q4cp_scale_stride.restype = C.c_uint64
        _lib.orc_q4cp_scale_stride.argtypes = [C.c_uint64]
        _lib.orc_q4cp_blob_bytes.restype = C.c_uint64
        _lib.orc_q4cp_blob_bytes.argtypes = [C.c_uint64, C.c_uint64]
        _lib.orc_q4k_row_bytes.restype = C.c_uint64
        _lib.orc_q4k_row_bytes.argtypes = [C.c_uint64]
        _lib.orc_num_threads.restype = C.c_int
        _lib.orc_gg_row_bytes.restype = C.c_uint64
        _lib.orc_gg_row_bytes.argtypes = [C.c_int, C.c_uint64]
    return _lib


def ref():
    """The reference's own code (oracle/_ref/libmoe_ref.so) or None when not built."""
    global _ref
    if _ref is None:
        path = os.path.join(_HERE, "_ref", "libmoe_ref.so")
        if not os.path.exists(path):
            return None
        _ref = C.CDLL(path)
        _ref.ref_fp16_to_f32.restype = C.c_float
        _ref.ref_fp16_to_f32.argtypes = [C.c_uint16]
        _ref.ref_q4k_row_bytes.restype = C.c_uint64
        _ref.ref_q4k_row_bytes.argtypes = [C.c_uint64]
        _ref.ref_gg_row_bytes.restype = C.c_uint64
        _ref.ref_gg_row_bytes.argtypes = [C.c_uint32, C.c_uint64]
    return _ref


def _p(a):
    return a.ctypes.data_as(C.c_void_p) if a is not None else None


def _c(a, dt):
    a = np.ascontiguousarray(a, dtype=dt)
    return a


class Mat:
    """A weight matrix in one of the supported storages; keeps its bytes alive."""

    def __init__(self, dtype, data, rows, cols):
        self.dtype, self.rows, self.cols = dtype, int(rows), int(cols)
        self.data = np.ascontiguousarray(data)
        if dtype == Q4CP:
            assert self.data.dtype == np.uint8 and self.data.size == lib().orc_q4cp_blob_bytes(rows, cols)
        elif dtype == Q4K:
            assert self.data.dtype == np.uint8 and self.data.size == rows * lib().orc_q4k_row_bytes(cols)
        elif dtype in GG_TYPES:
            assert self.data.dtype == np.uint8 and self.data.size == rows * lib().orc_gg_row_bytes(dtype, cols)
        elif dtype == F32:
            assert self.data.dtype == np.float32 and self.data.size == rows * cols
        elif dtype == BF16:
            assert self.data.dtype == np.uint16 and self.data.size == rows * cols
        elif dtype == Q8G64:
            assert self.data.dtype == np.uint8 and cols % 64 == 0 and self.data.size == rows * (cols + cols // 64 * 4)
        elif dtype == Q8G32:
            assert self.data.dtype == np.uint8 and cols % 32 == 0 and self.data.size == rows * cols + rows * cols // 32 * 2
        elif dtype == I4R:
            assert self.data.dtype == np.uint8 and cols % 128 == 0 and self.data.size == rows * cols // 2 + rows * cols // 128 * 2

    def c(self):
        return _Mat(self.dtype, self.data.ctypes.data, self.rows, self.cols)

    def dequant(self, row0=0, nrows=None):
        nrows = self.rows - row0 if nrows is None else nrows
        if self.dtype == Q4CP:
            return q4cp_rows(self.data, self.rows, self.cols, row0, nrows)
        if self.dtype == Q4K:
            rb = lib().orc_q4k_row_bytes(self.cols)
            return q4k_rows(self.data[row0 * rb:(row0 + nrows) * rb], nrows, self.cols)
        if self.dtype in GG_TYPES:
            rb = lib().orc_gg_row_bytes(self.dtype, self.cols)
            return gg_rows(self.dtype, self.data[row0 * rb:(row0 + nrows) * rb], nrows, self.cols)
        if self.dtype == F32:
            return self.data.reshape(self.rows, self.cols)[row0:row0 + nrows].copy()
        if self.dtype in (Q8G64, Q8G32, I4R):
            out = np.empty((nrows, self.cols), np.float32)
            m = self.c()
            lib().orc_mat_rows(C.byref(m), row0, nrows, _p(out))
            return out
        u = self.data.reshape(self.rows, self.cols)[row0:row0 + nrows].astype(np.uint32) << 16
        return u.view(np.float32)


_NULL = _Mat(-1, None, 0, 0)


def fp16_to_f32(h):
    return float(lib().orc_fp16_to_f32(int(h)))


def q4cp_rows(blob, rows, cols, row0, nrows):
    blob = _c(blob, np.uint8)
    out = np.empty((nrows, cols), np.float32)
    lib().orc_q4cp_rows(_p(blob), C.c_uint64(rows), C.c_uint64(cols), C.c_uint64(row0),
                        C.c_uint64(nrows), _p(out))
    return out


def gg_row_bytes(t, k):
    return int(lib().orc_gg_row_bytes(int(t), C.c_uint64(k)))


def gg_rows(t, raw, nrows, k):
    """Dequantised rows of a ggml block type (Q4_K, Q5_K, Q5_1, Q8_0), src/gguf.h:339-445."""
    raw = _c(raw, np.uint8)
    rb = gg_row_bytes(t, k)
    assert rb and raw.size == nrows * rb
    out = np.empty((nrows, k), np.float32)
    for r in range(nrows):
        rc = lib().orc_gg_row(int(t), C.c_void_p(raw.ctypes.data + r * rb), C.c_void_p(out.ctypes.data + r * k * 4),
                              C.c_uint64(k))
        assert rc == 0
    return out


def ref_gg_rows(t, raw, nrows, k):
    """The same through the reference's own gguf::dequant_row (oracle/_ref)."""
    raw = _c(raw, np.uint8)
    rb = int(ref().ref_gg_row_bytes(C.c_uint32(t), C.c_uint64(k)))
    assert raw.size == nrows * rb
    out = np.empty((nrows, k), np.float32)
    for r in range(nrows):
        rc = ref().ref_gg_row(C.c_uint32(t), C.c_void_p(raw.ctypes.data + r * rb),
                              C.c_void_p(out.ctypes.data + r * k * 4), C.c_uint64(k))
        assert rc == 0
    return out


def q4k_rows(raw, nrows, k):
    raw = _c(raw, np.uint8)
    rb = lib().orc_q4k_row_bytes(k)
    assert raw.size == nrows * rb
    out = np.empty((nrows, k), np.float32)
    for r in range(nrows):
        lib().orc_q4k_row(C.c_void_p(raw.ctypes.data + r * rb), C.c_void_p(out.ctypes.data + r * k * 4),
                          C.c_uint64(k))
    return out


def scale_min_k4(j, q12):
    q12 = _c(q12, np.uint8)
    d, m = C.c_uint8(), C.c_uint8()
    lib().orc_scale_min_k4(int(j), _p(q12), C.byref(d), C.byref(m))
    return d.value, m.value


def softmax_topk(logits, k):
    logits = _c(logits, np.float32)
    E = logits.size
    probs = np.empty(E, np.float32)
    ids = np.empty(k, np.int32)
    ws = np.empty(k, np.float32)
    lib().orc_softmax_topk(_p(logits), E, k, _p(probs), _p(ids), _p(ws))
    return probs, ids, ws


def router(Wr, x, k, bias=None, id_stride=16):
    """-> logits [T][E] f32, ids [T][id_stride] i32, ws [T][id_stride] f32 (first k valid)."""
    x = _c(x, np.float32).reshape(-1, Wr.cols)
    T, E = x.shape[0], Wr.rows
    logits = np.empty((T, E), np.float32)
    ids = np.zeros((T, id_stride), np.int32)
    ws = np.zeros((T, id_stride), np.float32)
    b = _c(bias, np.float32) if bias is not None else None
    m = Wr.c()
    lib().orc_router(C.byref(m), _p(b), _p(x), T, k, id_stride, _p(logits), _p(ids), _p(ws))
    return logits, ids, ws


def route(ids, ws, k, E):
    """Expert-sorted permutation -> tokidx, pw, eoff, pairids."""
    ids = _c(ids, np.int32)
    ws = _c(ws, np.float32)
    P, stride = ids.shape
    tokidx = np.empty(P * k, np.int32)
    pw = np.empty(P * k, np.float32)
    eoff = np.empty(E + 1, np.int32)
    pairids = np.empty(P * k, np.int32)
    lib().orc_route(_p(ids), _p(ws), P, k, E, stride, _p(tokidx), _p(pw), _p(eoff), _p(pairids))
    return tokidx, pw, eoff, pairids


def tiles(eoff, cap):
    eoff = _c(eoff, np.int32)
    E = eoff.size - 1
    out = np.empty((int(eoff[-1]) // cap + E + 1, 3), np.int32)
    lib().orc_tiles.restype = C.c_int
    n = lib().orc_tiles(_p(eoff), E, cap, _p(out))
    return out[:n].copy()


class Layer:
    """One MoE layer's weights for the oracle (numpy-backed)."""

    def __init__(self, d, mid, E, k, router, down, gate_up=None, gate=None, up=None,
                 shared=None, router_bias=None, rot=None):
        self.d, self.mid, self.E, self.k = d, mid, E, k
        # hgn v2 rotated experts: (su_gu [d], svh_gu [2 mid], suh_dn [mid], svh_dn [d]) as f32, else None
        self.rot = tuple(_c(a, np.float32) for a in rot) if rot is not None else None
        self.router, self.down, self.gate_up, self.gate, self.up = router, down, gate_up, gate, up
        self.shared = shared  # (sh_gate, sh_up, sh_down, sh_sg) or None
        self.router_bias = _c(router_bias, np.float32) if router_bias is not None else None

    def c(self):
        L = _Layer()
        L.d, L.mid, L.E, L.k = self.d, self.mid, self.E, self.k
        L.router = self.router.c()
        L.router_bias = self.router_bias.ctypes.data if self.router_bias is not None else None
        L.gate_up = self.gate_up.c() if self.gate_up is not None else _NULL
        L.gate = self.gate.c() if self.gate is not None else _NULL
        L.up = self.up.c() if self.up is not None else _NULL
        L.down = self.down.c()
        if self.shared is not None:
            L.sh_gate, L.sh_up, L.sh_down, L.sh_sg = (m.c() for m in self.shared)
            L.has_shared = 1
        else:
            L.sh_gate = L.sh_up = L.sh_down = L.sh_sg = _NULL
            L.has_shared = 0
        if self.rot is not None:
            L.su_gu, L.svh_gu, L.suh_dn, L.svh_dn = (a.ctypes.data for a in self.rot)
        return L


def moe_layer(layer, x, tok_list=None, id_stride=16, want_hid=False):
    """y [T][d] (rows outside tok_list are left NaN), ids, ws, hid?"""
    x = _c(x, np.float32).reshape(-1, layer.d)
    T = x.shape[0]
    ids = np.zeros((T, id_stride), np.int32)
    ws = np.zeros((T, id_stride), np.float32)
    y = np.full((T, layer.d), np.nan, np.float32)
    hid = np.full((T, layer.k, layer.mid), np.nan, np.float32) if want_hid else None
    tl = _c(tok_list, np.int32) if tok_list is not None else None
    L = layer.c()
    lib().orc_moe_layer(C.byref(L), _p(x), T, _p(tl), 0 if tl is None else tl.size, id_stride,
                        _p(ids), _p(ws), _p(hid), _p(y))
    return (y, ids, ws, hid) if want_hid else (y, ids, ws)


def v2_rot(x, pre=None, post=None):
    """post * H(pre * x) / sqrt(128) per block of 128 of every row (hgn v2 rotation)."""
    x = _c(x, np.float32)
    n = x.shape[-1]
    pre = _c(pre, np.float32) if pre is not None else None
    post = _c(post, np.float32) if post is not None else None
    out = np.empty_like(x)
    xr, orr = x.reshape(-1, n), out.reshape(-1, n)
    for i in range(xr.shape[0]):
        lib().orc_v2_rot(_p(xr[i]), _p(orr[i]), _p(pre), _p(post), n)
    return out


def ht_value(w16):
    lib().orc_ht_value.restype = C.c_float
    return lib().orc_ht_value(C.c_uint32(int(w16)))


def ht_decode(codes, rows, cols):
    """ht code stream -> its values G [rows][cols] in the rotated domain."""
    codes = _c(codes, np.uint8)
    assert codes.size == rows * cols // 2
    out = np.empty((rows, cols), np.float32)
    lib().orc_ht_decode(_p(codes), C.c_uint64(rows), C.c_uint64(cols), _p(out))
    return out


def v2_dense_bf16(dtype, data, rows, cols, suh=None, svh=None):
    """hgn v2 dense tensor (16 = ht with its planes as f32, 24 = q6g64) -> bf16 bits [rows][cols] (uint16)."""
    data = _c(data, np.uint8)
    out = np.empty((rows, cols), np.uint16)
    suh = _c(suh, np.float32) if suh is not None else None
    svh = _c(svh, np.float32) if svh is not None else None
    rc = lib().orc_v2_dense_bf16(int(dtype), _p(data), _p(suh), _p(svh), C.c_uint64(rows), C.c_uint64(cols), _p(out))
    assert rc == 0, rc
    return out


def num_threads():
    return lib().orc_num_threads()


def set_threads(n):
    lib().orc_set_threads(int(n))


# ---- the reference's own code (only where oracle/_ref is built) ----

def ref_q4cp_rows(blob, rows, cols, row0, nrows):
    blob = _c(blob, np.uint8)
    out = np.empty((nrows, cols), np.float32)
    rc = ref().ref_q4cp_rows(_p(blob), C.c_uint64(rows), C.c_uint64(cols), C.c_uint64(row0),
                             C.c_uint64(nrows), _p(out))
    assert rc == 0
    return out


def ref_dequant_tensor(mat):
    """Checkpoint::dequant of the reference on a BF16 / Q8G64 Mat."""
    out = np.empty((mat.rows, mat.cols), np.float32)
    rc = ref().ref_dequant_tensor(C.c_uint32(HGN_DTYPE[mat.dtype]), C.c_uint64(mat.rows), C.c_uint64(mat.cols),
                                  _p(mat.data), _p(out))
    assert rc == 0
    return out


def ref_q4k_rows(raw, nrows, k):
    raw = _c(raw, np.uint8)
    rb = ref().ref_q4k_row_bytes(C.c_uint64(k))
    out = np.empty((nrows, k), np.float32)
    for r in range(nrows):
        rc = ref().ref_q4k_row(C.c_void_p(raw.ctypes.data + r * rb),
                               C.c_void_p(out.ctypes.data + r * k * 4), C.c_uint64(k))
        assert rc == 0
    return out


def ref_scale_min_k4(j, q12):
    q12 = _c(q12, np.uint8)
    d, m = C.c_uint8(), C.c_uint8()
    ref().ref_scale_min_k4(int(j), _p(q12), C.byref(d), C.byref(m))
    return d.value, m.value


def ref_moe_token(layer, x):
    """Model::moe of the reference for one token.  Router/shared tensors must be BF16 or Q4CP,
    routed experts q4cp with fused gate_up."""
    x = _c(x, np.float32).reshape(layer.d)
    y = np.empty(layer.d, np.float32)
    sh_gate, sh_up, sh_down, sh_sg = layer.shared
    assert sh_gate.dtype == sh_up.dtype == sh_down.dtype
    rc = ref().ref_moe_token(layer.d, layer.mid, layer.E, layer.k, C.c_uint32(HGN_DTYPE[layer.router.dtype]),
                             _p(layer.router.data), _p(layer.gate_up.data), _p(layer.down.data),
                             C.c_uint32(HGN_DTYPE[sh_gate.dtype]), _p(sh_gate.data), _p(sh_up.data),
                             _p(sh_down.data), C.c_uint32(HGN_DTYPE[sh_sg.dtype]), _p(sh_sg.data), _p(x), _p(y))
    assert rc == 0
    return y


def _ref_tensor(fn, path, name):
    """-> (dtype, dims tuple, uint8 array) through one of the reference's file readers, or None."""
    dt, nd, nb = C.c_uint32(), C.c_uint32(), C.c_uint64()
    dims = (C.c_uint64 * 4)()
    rc = fn(str(path).encode(), name.encode(), C.byref(dt), C.byref(nd), dims, C.byref(nb), None, C.c_uint64(0))
    if rc == 1:
        return None
    if rc != 0:
        raise RuntimeError(f"reference reader failed on {path}")
    out = np.zeros(nb.value, np.uint8)
    fn(str(path).encode(), name.encode(), C.byref(dt), C.byref(nd), dims, C.byref(nb),
       out.ctypes.data_as(C.c_void_p), C.c_uint64(nb.value))
    return dt.value, tuple(dims[i] for i in range(nd.value)), out


def ref_hgn_tensor(path, name):
    """hgn::Checkpoint(path).find(name)  (src/hgn.h:103-106)"""
    return _ref_tensor(ref().ref_hgn_tensor, path, name)


def ref_gguf_tensor(path, name):
    """gguf::File(path).find(name)  (src/gguf.h:119-160)"""
    return _ref_tensor(ref().ref_gguf_tensor, path, name)


def ref_gguf_kv_i(path, key, default=-1):
    f = ref().ref_gguf_kv_i
    f.restype = C.c_int64
    return f(str(path).encode(), key.encode(), C.c_int64(default))


def layer_from_device(dl):
    """An oracle Layer over the very bytes of a synthetic device layer (an object with the attributes of
    gfx1151_engine_amd.workloads.DeviceLayer), copied to the host.  Checker side only."""
    d, mid, E, k = dl.d, dl.mid, dl.E, dl.k
    wt = Q4CP if dl.fmt == "q4cp" else I4R if dl.fmt == "i4r" else Q4K
    tgu, tdn, tsh = (getattr(dl, a, Q4K) for a in ("tgu", "tdn", "tsh"))  # ggml types of a raw-block layer
    st = Q4CP if dl.fmt in ("q4cp", "i4r") else tsh
    h = lambda t: t.cpu().numpy()
    sh = [Mat(st, h(dl.sh[0]), mid, d), Mat(st, h(dl.sh[1]), mid, d), Mat(st, h(dl.sh[2]), d, mid),
          Mat(F32, h(dl.sh_sg), 1, d)]
    router = Mat(F32, h(dl.router), E, d)
    bias = h(dl.bias) if dl.bias is not None else None
    if dl.fmt in ("q4cp", "i4r"):
        return Layer(d, mid, E, k, router, Mat(wt, h(dl.down), E * d, mid),
                     gate_up=Mat(wt, h(dl.gate_up), E * 2 * mid, d), shared=sh, router_bias=bias,
                     rot=[h(p) for p in dl.planes] if dl.fmt == "i4r" else None)
    return Layer(d, mid, E, k, router, Mat(tdn, h(dl.down), E * d, mid),
                 gate=Mat(tgu, h(dl.gate), E * mid, d), up=Mat(tgu, h(dl.up), E * mid, d),
                 shared=sh, router_bias=bias)


def hc_writeback(y, w4, R):
    """R (uint16 bf16 bits [P][4][D]) after the HC write-back of y (f32 [P][D]) with inject gate logits w4 [P][4]
    (src/gpu/parts/24_kernels_moe_lt.inc:126-161); returns a new array."""
    y = _c(y, np.float32)
    w4 = _c(w4, np.float32)
    out = np.ascontiguousarray(R, np.uint16).copy()
    P, D = y.shape
    assert w4.shape == (P, 4) and out.shape == (P, 4, D)
    lib().orc_hc_writeback(_p(y), _p(w4), _p(out), C.c_int(P), C.c_int(D))
    return out
