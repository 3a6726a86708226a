"""Writers for small synthetic checkpoint files in the engine's two formats (tests, examples).

  HGN1 (.hgn): 104-byte header, 160-byte tensor records, data  (reference: src/hgn.h:48-76,295-363)
  GGUF v3:      header, key-value section, tensor infos, aligned data  (reference: src/gguf.h:225-314)

The byte layouts of the tensors themselves are synth.make_q4cp / synth.make_q4k and plain bf16 / f32.
"""
import struct

import numpy as np

HGN_BF16, HGN_F32, HGN_Q4CP, HGN_Q8G64, HGN_Q8G32 = 0, 1, 5, 7, 8
HGN_F16, HGN_I4R = 2, 23  # hgn v2: f16 sign-scale planes, rotated routed experts
HGN_HT, HGN_Q6G64 = 16, 24  # hgn v2 dense tensors: hashed-trellis codes (with .suh / .svh planes), 6-bit groups of 64
GGML_F32, GGML_BF16, GGML_Q4_K = 0, 30, 12
_GGML_BLOCK = {0: (1, 4), 30: (1, 2), 1: (1, 2), 12: (256, 144), 13: (256, 176), 8: (32, 34), 7: (32, 24),
               20: (32, 18), 23: (256, 136)}


def _bytes(a):
    return np.ascontiguousarray(a).view(np.uint8).reshape(-1).tobytes()


def write_hgn(path, tensors, model_name="synthetic", align=64):
    """tensors: list of (name, dtype, dims, array of raw bytes).  dims are outermost first."""
    n = len(tensors)
    rec_off = 104
    data_off = (rec_off + 160 * n + align - 1) // align * align
    blobs, recs, off = [], [], data_off
    for name, dtype, dims, data in tensors:
        b = _bytes(data)
        assert len(name) < 96 and len(dims) <= 4
        d4 = list(dims) + [0] * (4 - len(dims))
        recs.append(struct.pack("<96sII4QQQQ", name.encode(), dtype, len(dims), *d4, off, len(b), 0))
        blobs.append((off, b))
        off = (off + len(b) + align - 1) // align * align
    size = off
    with open(path, "wb") as f:
        f.write(struct.pack("<4sIIIQQQ64s", b"HGN1", 1, n, 0, rec_off, data_off, size, model_name.encode()))
        for r in recs:
            f.write(r)
        for o, b in blobs:
            f.seek(o)
            f.write(b)
        f.truncate(size)


def _gguf_str(s):
    b = s.encode()
    return struct.pack("<Q", len(b)) + b


def write_gguf(path, tensors, kv=None, align=32):
    """tensors: list of (name, ggml type, ne (innermost first), raw bytes array).
    kv: dict of str -> int (written as uint32), str, float (float32) or list of str."""
    kv = dict(kv or {})
    out = [b"GGUF", struct.pack("<IQQ", 3, len(tensors), len(kv))]
    for k, v in kv.items():
        out.append(_gguf_str(k))
        if isinstance(v, bool):
            out.append(struct.pack("<IB", 7, int(v)))
        elif isinstance(v, int):
            out.append(struct.pack("<II", 4, v))
        elif isinstance(v, float):
            out.append(struct.pack("<If", 6, v))
        elif isinstance(v, str):
            out.append(struct.pack("<I", 8) + _gguf_str(v))
        else:  # list of strings
            out.append(struct.pack("<IIQ", 9, 8, len(v)) + b"".join(_gguf_str(x) for x in v))
    blobs, off = [], 0
    for name, typ, ne, data in tensors:
        b = _bytes(data)
        be, bb = _GGML_BLOCK[typ]
        assert int(np.prod(ne)) // be * bb == len(b), name
        out.append(_gguf_str(name) + struct.pack("<I", len(ne)) + struct.pack(f"<{len(ne)}Q", *ne) +
                   struct.pack("<IQ", typ, off))
        blobs.append((off, b))
        off = (off + len(b) + align - 1) // align * align
    hdr = b"".join(out)
    base = (len(hdr) + align - 1) // align * align
    with open(path, "wb") as f:
        f.write(hdr)
        for o, b in blobs:
            f.seek(base + o)
            f.write(b)
        f.truncate(base + off)


def hgn_layer_tensors(l, hl):
    """The MoE tensors of layer l of a tests.helpers.HostLayer-like object (fmt q4cp, or i4r = hgn v2 rotated experts
    with their four f16 planes under the reference's names, tools/v2repro/v2_encode.py:84-90) as .hgn records."""
    d, mid, E = hl.d, hl.mid, hl.E
    rdt = HGN_F32 if hl.router.dtype == np.float32 else HGN_BF16
    edt = HGN_I4R if getattr(hl, "fmt", "q4cp") == "i4r" else HGN_Q4CP
    t = [(f"layers.{l}.mlp.gate.weight", rdt, [E, d], hl.router),
         (f"layers.{l}.mlp.experts.gate_up_proj.weight", edt, [E, 2 * mid, d], hl.gate_up),
         (f"layers.{l}.mlp.experts.down_proj.weight", edt, [E, d, mid], hl.down)]
    if edt == HGN_I4R:
        su, svh_gu, suh_dn, svh_dn = (np.asarray(p, np.float32).astype(np.float16) for p in hl.planes)
        t += [(f"layers.{l}.mlp.experts.su", HGN_F16, [d], su),
              (f"layers.{l}.mlp.experts.gate_up_proj.svh", HGN_F16, [2 * mid], svh_gu),
              (f"layers.{l}.mlp.experts.down_proj.suh", HGN_F16, [mid], suh_dn),
              (f"layers.{l}.mlp.experts.down_proj.svh", HGN_F16, [d], svh_dn)]
    if hl.shared is not None:
        sdt = {None: HGN_Q4CP, "bf16": HGN_BF16, "f32": HGN_F32, "q8g64": HGN_Q8G64, "q8g32": HGN_Q8G32}[getattr(hl, "shared_dense", None)]
        t += [(f"layers.{l}.mlp.shared_expert.gate_proj.weight", sdt, [mid, d], hl.shared[0]),
              (f"layers.{l}.mlp.shared_expert.up_proj.weight", sdt, [mid, d], hl.shared[1]),
              (f"layers.{l}.mlp.shared_expert.down_proj.weight", sdt, [d, mid], hl.shared[2]),
              (f"layers.{l}.mlp.shared_expert_gate.weight", HGN_F32, [1, d], hl.shared[3])]
    return t


def gguf_layer_tensors(l, hl):
    """The MoE tensors of layer l of a HostLayer-like object (fmt q4k; ggml types hl.tgu / hl.tdn / hl.tsh where
    it has them, else Q4_K) as GGUF tensor infos."""
    d, mid, E = hl.d, hl.mid, hl.E
    tgu, tdn, tsh = (getattr(hl, a, GGML_Q4_K) for a in ("tgu", "tdn", "tsh"))
    t = [(f"blk.{l}.ffn_gate_inp.weight", GGML_F32, [d, E], hl.router),
         (f"blk.{l}.ffn_gate_exps.weight", tgu, [d, mid, E], hl.gate),
         (f"blk.{l}.ffn_up_exps.weight", tgu, [d, mid, E], hl.up),
         (f"blk.{l}.ffn_down_exps.weight", tdn, [mid, d, E], hl.down)]
    if hl.shared is not None:
        t += [(f"blk.{l}.ffn_gate_shexp.weight", tsh, [d, mid], hl.shared[0]),
              (f"blk.{l}.ffn_up_shexp.weight", tsh, [d, mid], hl.shared[1]),
              (f"blk.{l}.ffn_down_shexp.weight", tsh, [mid, d], hl.shared[2]),
              (f"blk.{l}.ffn_gate_inp_shexp.weight", GGML_F32, [d], hl.shared[3])]
    return t
